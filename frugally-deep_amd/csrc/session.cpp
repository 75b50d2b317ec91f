// Autoregressive decoding over a loaded decoder model: causal self-attention with the
// projected keys / values of every layer cached in HBM (token-major, so a new token's
// projection GEMM writes its cache row in place).
//
// The reference has neither a mask nor a cache (include/fdeep/layers/multi_head_attention_layer.hpp:74-95).
// A session position t is defined through a call the reference does support,
// MultiHeadAttention(query = x[t:t+1], value = x[0:t+1]) (same file, :98-103): every op of the model
// other than attention works on rows independently, so caching K/V of earlier rows and attending the
// new rows to the visible prefix computes exactly that.
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <map>

#include "model.hpp"
#include "skinny.hpp"

using namespace fdx;

struct fdx_session {
    fdx_model* m = nullptr;
    int batch = 0, max_len = 0, len = 0;
    std::vector<int> order;
    int last_mha_pos = -1;
    int vocab = 0;
    std::map<int, float*> kc, vc; // per MultiHeadAttention op
    // bump arena for activations of one call; chunks are kept and reused by later calls
    struct Chunk {
        void* p;
        size_t bytes, used;
    };
    std::vector<Chunk> chunks;

    // ---- decode fast path (one new token per sequence, batch <= 16): a fixed list of fused launches
    // over buffers allocated once; built at creation when the graph has the expected decoder structure
    struct Step {
        enum Kind { EmbedAdd, Gemm, Attn, AttnProj, LayerNorm, Add, Act, Softmax } kind;
        SkinnyParams g;                 // Gemm
        const float *a = nullptr, *b = nullptr; // operands of the other kinds
        float* out = nullptr;
        int op = -1;                    // model op this step realises
        int depth = 0;
        // AttnProj: the output projection that rides in the attention launch
        const float* proj_w = nullptr;  // [heads][64][depth]
        const float* proj_bias = nullptr;
        const float* proj_residual = nullptr;
        fdx::Act proj_act { FDX_ACT_NONE, 3.402823466e+38f, 0.f, 0.f };
        int mha_op = -1;
    };
    bool fast = false;
    std::vector<Step> steps;
    std::vector<void*> owned;           // device buffers of the fast path
    int* len_dev = nullptr;             // tokens already cached, read by the fast-path kernels
    float* ids_buf = nullptr;           // ids consumed by the next step (argmax writes them)
    const float* logits_buf = nullptr;
    unsigned long long* amax = nullptr; // per sequence: packed running arg-max of the step's logits
    unsigned long long* amax_parts = nullptr; // [workgroups of the logits launch][16] when that launch leaves partial maxima
    int amax_part_count = 0;
    float* history = nullptr;           // [max_len][batch] greedy ids by the position that produced them
    hipGraphExec_t step_graph = nullptr; // one decode step (ids_buf -> ids_buf) captured for replay
    hipGraphExec_t step_graph_merged = nullptr; // the same without the embedding launch, its last launch embedding the picked ids
    float* splitk_ws = nullptr;         // per-head partial rows of the attention + projection launches
    int* splitk_tickets = nullptr;      // their tickets, one per sequence, zero between launches
    static constexpr int64_t kWsFloats = 1 << 20;
    static constexpr int kTickets = 4096;
    float* positions = nullptr;
    ~fdx_session()
    {
        (void)hipStreamSynchronize(stream());

        for (auto& c : chunks)
            (void)hipFree(c.p);
        for (auto& kv : kc)
            (void)hipFree(kv.second);
        for (auto& kv : vc)
            (void)hipFree(kv.second);
        for (void* p : owned)
            (void)hipFree(p);
        if (step_graph)
            (void)hipGraphExecDestroy(step_graph);
        if (step_graph_merged)
            (void)hipGraphExecDestroy(step_graph_merged);
    }
    void arena_reset()
    {
        for (auto& c : chunks)
            c.used = 0;
    }
    float* arena(size_t bytes)
    {
        bytes = (bytes + 255) & ~(size_t)255;
        for (auto& c : chunks)
            if (c.bytes - c.used >= bytes) {
                float* r = reinterpret_cast<float*>(static_cast<char*>(c.p) + c.used);
                c.used += bytes;
                return r;
            }
        Chunk c { nullptr, std::max(bytes, (size_t)64 << 20), 0 };
        if (hipMalloc(&c.p, c.bytes) != hipSuccess)
            return nullptr;
        c.used = bytes;
        chunks.push_back(c);
        return static_cast<float*>(c.p);
    }
};

static int g_embed_fold = -1; // test hook: -1 = the environment decides, 0 / 1 = sessions created from now on

extern "C" fdx_status fdx_debug_decode_embed_fold(int mode)
{
    FDX_REQUIRE(mode >= -1 && mode <= 1, "fdx_debug_decode_embed_fold: mode must be -1, 0 or 1");
    g_embed_fold = mode;
    return FDX_OK;
}

namespace {

fdx_act to_c(const Act& a) { return { a.kind, a.max_value, a.negative_slope, a.threshold }; }

int depth_of(const fdx_model& m, int idx, std::vector<int>& memo)
{
    if (memo[idx] >= 0)
        return memo[idx];
    const Op& o = m.ops[idx];
    int d = 1;
    switch (o.kind) {
    case OpKind::Input: d = 1; break;
    case OpKind::Embedding: d = o.output_dim; break;
    case OpKind::Dense: d = o.units; break;
    case OpKind::MHA: d = o.dout; break;
    default: d = depth_of(m, o.in[0], memo); break;
    }
    return memo[idx] = d;
}

// T new tokens per sequence: ids_dev [batch][T]
fdx_status run(fdx_session* s, const float* ids_dev, int T, float* logits_dev, float* next_ids_dev)
{
    fdx_model& m = *s->m;
    FDX_REQUIRE(ids_dev && T > 0, "session: bad arguments");
    FDX_REQUIRE(s->len + T <= s->max_len, "session: sequence length %d exceeds max_len %d", s->len + T, s->max_len);
    std::lock_guard<std::mutex> lock(m.mu);
    const int B = s->batch;
    s->arena_reset();
    std::vector<float*> buf(m.ops.size(), nullptr);
    std::vector<int64_t> rows(m.ops.size(), 0);
    std::vector<int> dmemo(m.ops.size(), -1);
    std::map<int, float*> gathered; // last-row copies of tensors produced at full length
    fdx_status st = FDX_OK;

    float* pos = s->arena(sizeof(float) * (size_t)B * T);
    if (!pos) {
        set_error("session: out of device memory");
        return FDX_ERR_HIP;
    }
    if ((st = positions_launch(pos, B, T, s->len)) != FDX_OK)
        return st;

    for (size_t p = 0; p < s->order.size(); ++p) {
        const int idx = s->order[p];
        const Op& o = m.ops[idx];
        if (o.dead)
            continue;
        const bool tail = (int)p > s->last_mha_pos && T > 1; // only the last position of every sequence is needed
        const int64_t R = tail ? B : (int64_t)B * T;
        // operands at the row count this op works on
        auto operand = [&](int src) -> const float* {
            if (rows[src] == R)
                return buf[src];
            auto it = gathered.find(src);
            if (it != gathered.end())
                return it->second;
            const int d = depth_of(m, src, dmemo);
            float* g = s->arena(sizeof(float) * (size_t)B * d);
            if (!g)
                return nullptr;
            if (gather_rows_launch(buf[src], B, d, (int64_t)T * d, (int64_t)(T - 1) * d, g) != FDX_OK)
                return nullptr;
            gathered[src] = g;
            return g;
        };
        const int depth = depth_of(m, idx, dmemo);
        const fdx_act act = to_c(o.act);
        const fdx_act* actp = o.act.kind == FDX_ACT_NONE ? nullptr : &act;
        rows[idx] = R;
        if (o.kind == OpKind::Input) {
            buf[idx] = o.input_index == 0 ? const_cast<float*>(ids_dev) : pos;
            rows[idx] = (int64_t)B * T;
            continue;
        }
        const float* in0 = operand(o.in[0]);
        const float* res = o.residual >= 0 ? operand(o.residual) : nullptr;
        if (!in0 || (o.residual >= 0 && !res)) {
            set_error("session: out of device memory");
            return FDX_ERR_HIP;
        }
        if (o.kind == OpKind::View) {
            buf[idx] = const_cast<float*>(in0);
            continue;
        }
        float* out = s->arena(sizeof(float) * (size_t)R * depth);
        if (!out) {
            set_error("session: out of device memory");
            return FDX_ERR_HIP;
        }
        buf[idx] = out;
        switch (o.kind) {
        case OpKind::Embedding:
            st = fdx_embedding_f32(in0, R, o.dw[0], o.input_dim, o.output_dim, out, m.err_flag);
            break;
        case OpKind::Add: {
            const float* acc = in0;
            for (size_t k = 1; k < o.in.size() && st == FDX_OK; ++k) {
                const float* b = operand(o.in[k]);
                if (!b) {
                    set_error("session: out of device memory");
                    return FDX_ERR_HIP;
                }
                st = fdx_eltwise_add_f32(acc, b, (size_t)R * depth, (size_t)R * depth, k + 1 == o.in.size() ? actp : nullptr, out);
                acc = out;
            }
            break;
        }
        case OpKind::LayerNorm:
            st = fdx_layernorm_f32(in0, R, depth, o.dw[0], o.dw[1], o.eps, out);
            break;
        case OpKind::Act:
            st = fdx_activation_f32(in0, (size_t)R * depth, actp, out);
            break;
        case OpKind::Softmax:
            st = fdx_softmax_f32(in0, R, depth, 0, 0, out);
            break;
        case OpKind::Dense:
            st = fdx_gemm_bias_act_f32(in0, o.n_in, o.dw[0], o.n_in, (int)R, o.units, o.n_in, 1.f, o.dw[1], 0, res, actp, out, o.units,
                nullptr);
            if (st == FDX_OK && o.softmax)
                st = fdx_softmax_f32(out, R, o.units, 0, 0, out);
            break;
        case OpKind::MHA: {
            const int H = o.heads, D = o.d_in;
            const int64_t nk = (int64_t)H * o.dk, nv = (int64_t)H * o.dv;
            float* kc = s->kc[idx];
            float* vc = s->vc[idx];
            float* q = s->arena(sizeof(float) * (size_t)R * nk);
            float* merged = s->arena(sizeof(float) * (size_t)R * nv);
            if (!q || !merged) {
                set_error("session: out of device memory");
                return FDX_ERR_HIP;
            }
            if ((st = fdx_gemm_bias_act_f32(in0, D, o.dw[0], D, (int)R, (int)nk, D, 1.f, o.dw[1], 0, nullptr, nullptr, q, nk, nullptr)) != FDX_OK)
                return st;
            // keys / values of the new tokens go straight into their cache rows
            float* kdst = kc + (int64_t)s->len * nk;
            float* vdst = vc + (int64_t)s->len * nv;
            if (T == 1) {
                st = fdx_gemm_bias_act_f32(in0, D, o.dw[2], D, B, (int)nk, D, 1.f, o.dw[3], 0, nullptr, nullptr, kdst, (int64_t)s->max_len * nk, nullptr);
                if (st == FDX_OK)
                    st = fdx_gemm_bias_act_f32(in0, D, o.dw[4], D, B, (int)nv, D, 1.f, o.dw[5], 0, nullptr, nullptr, vdst, (int64_t)s->max_len * nv, nullptr);
                if (st == FDX_OK)
                    st = fdx_mha_decode_f32(q, kc, vc, B, H, o.dk, o.dv, s->len + 1, s->max_len, merged);
            } else {
                fdx_gemm_batch bt {};
                bt.batch = B;
                bt.inner = 1;
                bt.a_outer = (int64_t)T * D;
                bt.c_outer = (int64_t)s->max_len * nk;
                st = fdx_gemm_bias_act_f32(in0, D, o.dw[2], D, T, (int)nk, D, 1.f, o.dw[3], 0, nullptr, nullptr, kdst, nk, &bt);
                bt.c_outer = (int64_t)s->max_len * nv;
                if (st == FDX_OK)
                    st = fdx_gemm_bias_act_f32(in0, D, o.dw[4], D, T, (int)nv, D, 1.f, o.dw[5], 0, nullptr, nullptr, vdst, nv, &bt);
                if (st == FDX_OK) {
                    const int S = s->len + T;
                    void* scratch = s->arena(fdx_mha_scratch_bytes(B, H, T, S, o.dv));
                    if (!scratch) {
                        set_error("session: out of device memory");
                        return FDX_ERR_HIP;
                    }
                    st = mha_prefill_strided(q, nk, (int64_t)T * nk, kc, nk, (int64_t)s->max_len * nk, vc, nv, (int64_t)s->max_len * nv, B, T, S,
                        H, o.dk, o.dv, 1, merged, nv, (int64_t)T * nv, scratch);
                }
            }
            if (st == FDX_OK)
                st = fdx_gemm_bias_act_f32(merged, nv, o.dw[6], nv, (int)R, o.dout, (int)nv, 1.f, o.dw[7], 0, res, actp, out, o.dout,
                    nullptr);
            break;
        }
        default:
            set_error("session: layer %s (%s) is not a per-position op", o.name.c_str(), o.cls.c_str());
            return FDX_ERR_UNSUPPORTED;
        }
        if (st != FDX_OK)
            return st;
    }
    const int out_idx = m.outputs[0];
    const float* logits = buf[out_idx];
    if (rows[out_idx] != B) { // no attention layer after which to cut, or T == 1 handled above: take last rows
        float* g = s->arena(sizeof(float) * (size_t)B * s->vocab);
        if (!g || gather_rows_launch(logits, B, s->vocab, (int64_t)T * s->vocab, (int64_t)(T - 1) * s->vocab, g) != FDX_OK) {
            set_error("session: out of device memory");
            return FDX_ERR_HIP;
        }
        logits = g;
    }
    if (logits_dev)
        FDX_HIP(hipMemcpyAsync(logits_dev, logits, sizeof(float) * (size_t)B * s->vocab, hipMemcpyDeviceToDevice, stream()));
    if (next_ids_dev)
        if ((st = argmax_launch(logits, B, s->vocab, nullptr, nullptr, next_ids_dev)) != FDX_OK)
            return st;
    s->len += T;
    return FDX_OK;
}

// ---------------------------------------------------------------- decode fast path
// Turns the op list into fused decode launches: token+position embedding in one kernel; a
// LayerNorm that only feeds Dense / attention layers becomes the prologue of their weight-
// streaming GEMM; q, k and v come from one GEMM that writes the new cache rows in place; the
// residual Add after attention rides in the output projection's epilogue.  Returns false (and
// leaves the generic path in charge) when the graph does not have that structure.
bool build_fast_plan(fdx_session* s)
{
    fdx_model& m = *s->m;
    const int B = s->batch;
    if (B > 16)
        return false;
    std::vector<int> dmemo(m.ops.size(), -1);
    std::vector<float*> buf(m.ops.size(), nullptr);
    std::vector<int> lazy_ln(m.ops.size(), -1); // LayerNorm op applied inside its consumers' GEMMs
    std::vector<int> consumers(m.ops.size(), 0);
    std::vector<std::vector<int>> users(m.ops.size());
    for (int idx : s->order) {
        const Op& o = m.ops[idx];
        if (o.dead)
            continue;
        for (int i : o.in)
            users[i].push_back(idx);
        if (o.residual >= 0)
            users[o.residual].push_back(idx);
    }
    // Every buffer of the decode step comes out of a few large allocations: hundreds of separate small ones would each sit
    // on pages of their own, and a launch that touches a dozen operands would miss the address translation caches for
    // most of them.
    char* chunk = nullptr;
    size_t chunk_left = 0;
    auto alloc = [&](size_t floats) -> float* {
        const size_t bytes = (floats * sizeof(float) + 255) & ~(size_t)255;
        if (bytes > chunk_left) {
            // 32 MiB first, doubling up to 256 MiB: a small model's session stays small, a large one still ends up in a
            // handful of allocations
            const size_t step = std::min((size_t)256 << 20, (size_t)32 << 20 << std::min<size_t>(s->owned.size(), 3));
            const size_t want = std::max(bytes, step);
            void* p = nullptr;
            if (hipMalloc(&p, want) != hipSuccess)
                return nullptr;
            s->owned.push_back(p);
            chunk = static_cast<char*>(p);
            chunk_left = want;
        }
        float* r = reinterpret_cast<float*>(chunk);
        chunk += bytes;
        chunk_left -= bytes;
        return r;
    };
    s->len_dev = reinterpret_cast<int*>(alloc(1));
    if (!s->len_dev)
        return false;
    s->ids_buf = alloc((size_t)B);
    s->amax = reinterpret_cast<unsigned long long*>(alloc((size_t)2 * B + 4));
    if (!s->ids_buf || !s->amax)
        return false;
    if (zero_device(s->amax, sizeof(unsigned long long) * B) != hipSuccess)
        return false;
    s->history = alloc((size_t)s->max_len * B);
    if (!s->history || skinny_prepare() != FDX_OK)
        return false;
    s->splitk_ws = alloc((size_t)fdx_session::kWsFloats);
    s->splitk_tickets = reinterpret_cast<int*>(alloc((size_t)fdx_session::kTickets));
    if (!s->splitk_ws || !s->splitk_tickets || zero_device(s->splitk_tickets, sizeof(int) * fdx_session::kTickets) != hipSuccess)
        return false;
    std::vector<char> skip(m.ops.size(), 0);
    const int ids_op = m.inputs[0], pos_op = m.inputs[1];

    for (int idx : s->order) {
        const Op& o = m.ops[idx];
        if (o.dead || skip[idx] || o.kind == OpKind::Input)
            continue;
        const int depth = depth_of(m, idx, dmemo);
        fdx_session::Step st;
        st.op = idx;
        st.depth = depth;
        // operand of a weight-streaming GEMM; a pending LayerNorm is folded into copies of the weights
        // (W * gamma, row sums, bias + W beta) so the launch works on the raw rows
        auto gemm_input = [&](int src, SkinnyParams& g, const float* w, const float* bias, int n, int k) -> bool {
            g.W = w;
            g.bias = bias;
            if (lazy_ln[src] < 0) {
                g.X = buf[src];
                g.ln = 0;
                return g.X != nullptr;
            }
            const Op& ln = m.ops[src];
            float* wf = alloc((size_t)n * k);
            float* ws = alloc((size_t)n);
            float* bf = alloc((size_t)n);
            if (!wf || !ws || !bf || fold_layernorm_launch(ln.dw[0], ln.dw[1], w, bias, n, k, wf, ws, bf) != FDX_OK)
                return false;
            g.X = buf[ln.in[0]];
            g.ln = 1;
            g.ln_eps = ln.eps;
            g.W = wf;
            g.w_rowsum = ws;
            g.bias = bf;
            return g.X != nullptr;
        };
        switch (o.kind) {
        case OpKind::View:
            buf[idx] = buf[o.in[0]];
            continue;
        case OpKind::Embedding: {
            // only as one half of Add(Embedding(ids), Embedding(positions))
            if (users[idx].size() != 1)
                return false;
            const Op& add = m.ops[users[idx][0]];
            if (add.kind != OpKind::Add || add.in.size() != 2 || add.act.kind != FDX_ACT_NONE)
                return false;
            const Op& ea = m.ops[add.in[0]];
            const Op& eb = m.ops[add.in[1]];
            if (ea.kind != OpKind::Embedding || eb.kind != OpKind::Embedding || users[add.in[0]].size() != 1
                || users[add.in[1]].size() != 1 || ea.output_dim != eb.output_dim)
                return false;
            const bool a_is_ids = ea.in[0] == ids_op && eb.in[0] == pos_op;
            const bool b_is_ids = eb.in[0] == ids_op && ea.in[0] == pos_op;
            if (!a_is_ids && !b_is_ids)
                return false;
            if (idx != add.in[0])
                continue; // emitted when the first operand is visited
            const Op& tok = a_is_ids ? ea : eb;
            const Op& pos = a_is_ids ? eb : ea;
            st.kind = fdx_session::Step::EmbedAdd;
            st.a = tok.dw[0];
            st.b = pos.dw[0];
            st.g.M = tok.input_dim;
            st.g.N = pos.input_dim;
            st.depth = tok.output_dim;
            st.out = alloc((size_t)B * tok.output_dim);
            if (!st.out)
                return false;
            st.op = users[idx][0];
            buf[st.op] = st.out;
            skip[st.op] = 1;
            s->steps.push_back(st);
            continue;
        }
        case OpKind::LayerNorm: {
            bool all_gemm = !users[idx].empty() && o.target_shape.size() == 1 && depth <= 1024 && depth % 4 == 0;
            for (int u : users[idx]) {
                const Op& c = m.ops[u];
                const bool feeds_gemm = (c.kind == OpKind::Dense && c.in[0] == idx && c.residual != idx)
                    || (c.kind == OpKind::MHA);
                all_gemm = all_gemm && feeds_gemm;
            }
            for (int out : m.outputs)
                all_gemm = all_gemm && out != idx;
            if (all_gemm) {
                lazy_ln[idx] = o.in[0];
                continue;
            }
            st.kind = fdx_session::Step::LayerNorm;
            st.a = buf[o.in[0]];
            break;
        }
        case OpKind::Dense: {
            st.kind = fdx_session::Step::Gemm;
            SkinnyParams& g = st.g;
            std::memset(&g, 0, sizeof g);
            if (!gemm_input(o.in[0], g, o.dw[0], o.dw[1], o.units, o.n_in))
                return false;
            g.ldx = o.n_in;
            g.ldw = o.n_in;
            g.M = B;
            g.N = o.units;
            g.K = o.n_in;
            g.act = o.act;
            if (o.residual >= 0) {
                if (lazy_ln[o.residual] >= 0)
                    return false;
                g.residual = buf[o.residual];
                g.ldr = o.units;
            }
            if (o.softmax)
                return false;
            break;
        }
        case OpKind::MHA: {
            const int H = o.heads, D = o.d_in;
            const int nk = H * o.dk, nv = H * o.dv, nqkv = 2 * nk + nv;
            // fused projection weights [q | k | v][D] and bias
            float* wqkv = alloc((size_t)nqkv * D);
            float* bqkv = alloc((size_t)nqkv);
            float* q = alloc((size_t)B * nk);
            float* merged = alloc((size_t)B * nv);
            if (!wqkv || !bqkv || !q || !merged)
                return false;
            const size_t f = sizeof(float);
            // on the library stream, like the launches that read the copies (a plain device-to-device hipMemcpy runs on the
            // null stream, which this stream does not wait for, and may return before the copy has happened)
            hipStream_t cs = stream();
            if (hipMemcpyAsync(wqkv, o.dw[0], f * nk * D, hipMemcpyDeviceToDevice, cs) != hipSuccess
                || hipMemcpyAsync(wqkv + (size_t)nk * D, o.dw[2], f * nk * D, hipMemcpyDeviceToDevice, cs) != hipSuccess
                || hipMemcpyAsync(wqkv + (size_t)2 * nk * D, o.dw[4], f * nv * D, hipMemcpyDeviceToDevice, cs) != hipSuccess
                || hipMemcpyAsync(bqkv, o.dw[1], f * nk, hipMemcpyDeviceToDevice, cs) != hipSuccess
                || hipMemcpyAsync(bqkv + nk, o.dw[3], f * nk, hipMemcpyDeviceToDevice, cs) != hipSuccess
                || hipMemcpyAsync(bqkv + 2 * nk, o.dw[5], f * nv, hipMemcpyDeviceToDevice, cs) != hipSuccess)
                return false;
            fdx_session::Step pr;
            pr.kind = fdx_session::Step::Gemm;
            pr.op = idx;
            SkinnyParams& g = pr.g;
            std::memset(&g, 0, sizeof g);
            if (!gemm_input(o.in[0], g, wqkv, bqkv, nqkv, D))
                return false;
            g.ldx = D; g.ldw = D; g.M = B; g.N = nqkv; g.K = D;
            g.act = Act { FDX_ACT_NONE, 3.402823466e+38f, 0.f, 0.f };
            g.n_seg = 3;
            g.seg[0] = { q, nk, 0, 0 };
            g.seg[1] = { s->kc[idx], (int64_t)s->max_len * nk, nk, nk };
            g.seg[2] = { s->vc[idx], (int64_t)s->max_len * nv, 2 * nk, nv };
            g.len_dev = s->len_dev;
            s->steps.push_back(pr);
            // output projection; a following two-input Add becomes its residual operand
            st.kind = fdx_session::Step::Gemm;
            SkinnyParams& og = st.g;
            std::memset(&og, 0, sizeof og);
            og.X = merged; og.ldx = nv; og.W = o.dw[6]; og.ldw = nv; og.M = B; og.N = o.dout; og.K = nv; og.bias = o.dw[7];
            og.act = Act { FDX_ACT_NONE, 3.402823466e+38f, 0.f, 0.f };
            if (o.residual >= 0) { // the Add behind the attention was folded into it at load
                if (lazy_ln[o.residual] >= 0 || !buf[o.residual])
                    return false;
                og.residual = buf[o.residual];
                og.ldr = o.dout;
                og.act = o.act;
            }
            bool is_output = false;
            for (int out : m.outputs)
                is_output = is_output || out == idx;
            if (!is_output && users[idx].size() == 1 && o.residual < 0) {
                const int ai = users[idx][0];
                const Op& add = m.ops[ai];
                if (add.kind == OpKind::Add && add.in.size() == 2 && add.in[0] != add.in[1]) {
                    const int other = add.in[0] == idx ? add.in[1] : add.in[0];
                    if (buf[other] && lazy_ln[other] < 0) {
                        og.residual = buf[other];
                        og.ldr = o.dout;
                        og.act = add.act;
                        st.op = ai;
                        skip[ai] = 1;
                    }
                }
            }
            // Attention and this projection as one launch where the kernel covers the shape: one dependent launch less
            // per block, against an exchange of per-head partial rows between workgroups that costs about half a launch
            // itself.  Measured on the GPT-2-small shape (batch 16): 0.498 ms per step against 0.484 ms for the two
            // launches, so it is off unless FDX_DECODE_FUSE_PROJ=1 is set when the session is created.
            const char* fuse_env = std::getenv("FDX_DECODE_FUSE_PROJ");
            const bool fuse_proj = fuse_env && fuse_env[0] == '1';
            const bool act_ok = og.act.kind == FDX_ACT_NONE || og.act.kind == FDX_ACT_RELU || og.act.kind == FDX_ACT_GELU;
            if (fuse_proj && act_ok
                && mha_decode_proj_supported(B, H, o.dk, o.dv, s->max_len, nk, o.dout, fdx_session::kWsFloats, fdx_session::kTickets)) {
                float* wt = alloc((size_t)H * o.dout * 64);
                if (!wt || pack_proj_heads_launch(o.dw[6], H, o.dout, wt) != FDX_OK)
                    return false;
                st.kind = fdx_session::Step::AttnProj;
                st.a = q;
                st.proj_w = wt;
                st.proj_bias = o.dw[7];
                st.proj_residual = og.residual;
                st.proj_act = og.act;
                st.mha_op = idx;
                std::memset(&og, 0, sizeof og);
            } else {
                fdx_session::Step at;
                at.kind = fdx_session::Step::Attn;
                at.op = idx;
                at.a = q;
                at.out = merged;
                s->steps.push_back(at);
            }
            break;
        }
        case OpKind::Add:
            if (o.in.size() != 2 || lazy_ln[o.in[0]] >= 0 || lazy_ln[o.in[1]] >= 0)
                return false;
            st.kind = fdx_session::Step::Add;
            st.a = buf[o.in[0]];
            st.b = buf[o.in[1]];
            break;
        case OpKind::Act:
            st.kind = fdx_session::Step::Act;
            st.a = buf[o.in[0]];
            break;
        case OpKind::Softmax:
            st.kind = fdx_session::Step::Softmax;
            st.a = buf[o.in[0]];
            break;
        default:
            return false;
        }
        if (st.kind != fdx_session::Step::Gemm && !st.a)
            return false;
        if (st.kind == fdx_session::Step::Gemm && !st.g.X)
            return false;
        st.out = alloc((size_t)B * st.depth);
        if (!st.out)
            return false;
        if (st.kind == fdx_session::Step::Gemm) {
            st.g.n_seg = 1;
            st.g.seg[0] = { st.out, st.g.N, 0, 0 };
            st.g.len_dev = s->len_dev;
        }
        buf[st.op] = st.out;
        if (st.op != idx)
            buf[idx] = st.out;
        s->steps.push_back(st);
    }
    for (auto& stp : s->steps)
        if (stp.kind == fdx_session::Step::Gemm) {
            // decode-time copy of the operand in the order the kernel's lanes read it; narrow or long-K
            // projections without LayerNorm stay row-major because they run split along K instead
            const bool split_candidate = !stp.g.ln && stp.g.K > 1024;
            if (!split_candidate) {
                float* packed = alloc((size_t)packed_weight_floats(stp.g.N, stp.g.K));
                if (!packed || pack_weights_launch(stp.g.W, stp.g.N, stp.g.K, stp.g.ldw, packed) != FDX_OK)
                    return false;
                stp.g.W = packed;
                stp.g.packed = 1;
            }
            stp.g.workspace = nullptr; // launches that split K take the library's workspace and tickets
            stp.g.workspace_floats = fdx_session::kWsFloats;
            stp.g.tickets = s->splitk_tickets;
            stp.g.ticket_count = fdx_session::kTickets;
        }
    s->logits_buf = buf[m.outputs[0]];
    if (!s->logits_buf || lazy_ln[m.outputs[0]] >= 0)
        return false;
    // the embedding launch opens every step and clears the packed arg-max cells the last launch fills
    if (s->steps.empty() || s->steps.front().kind != fdx_session::Step::EmbedAdd)
        return false;
    // a vocabulary-sized logits launch leaves per-workgroup maxima next to the logits, which saves the pass over them
    if (s->steps.back().kind == fdx_session::Step::Gemm && s->steps.back().g.n_seg == 1 && s->steps.back().g.seg[0].ptr == s->logits_buf && s->batch <= 16) {
        SkinnyParams& g = s->steps.back().g;
        const int parts = skinny_wide_grid(g);
        if (parts > 0) {
            s->amax_parts = reinterpret_cast<unsigned long long*>(alloc((size_t)parts * 16 * 2));
            if (!s->amax_parts)
                return false;
            g.amax_parts = s->amax_parts;
            s->amax_part_count = parts;
        }
    }
    // The embedding launch itself goes where its result has two readers only, the first projection GEMM (through its
    // folded LayerNorm) and the residual operand of the GEMM behind the first attention: both form the rows from the two
    // tables on the way in, which takes one launch off the step's chain.  (The packed arg-max cells that launch clears
    // are not used when the logits launch leaves per-workgroup maxima.)  Measured on the GPT-2-small shape at batch 16 the
    // step gets 2.5 us longer, not shorter: the launch saved is 4.9 us, but each of the two GEMMs now starts with a
    // dependent chain of its own (id, then row) in front of loads that used to be independent.  Hence off unless
    // FDX_DECODE_EMBED_FOLD=1 is set or fdx_debug_decode_embed_fold(1) was called when the session is created.
    const char* fold_env = std::getenv("FDX_DECODE_EMBED_FOLD");
    const bool fold_on = g_embed_fold > 0 || (g_embed_fold < 0 && fold_env && fold_env[0] == '1');
    if (fold_on && s->amax_part_count > 0 && s->steps.size() > 2) {
        const fdx_session::Step emb = s->steps.front();
        const float* x0 = emb.out;
        int as_x = 0, as_res = 0;
        bool other = x0 == s->logits_buf;
        for (size_t i = 1; i < s->steps.size(); ++i) {
            const auto& st = s->steps[i];
            if (st.kind == fdx_session::Step::Gemm) {
                const bool plain = skinny_wide_grid(st.g) == 0 && st.g.K <= 1024;
                if (st.g.X == x0) {
                    ++as_x;
                    other = other || !plain || st.g.K != emb.depth || st.g.ldx != emb.depth;
                }
                if (st.g.residual == x0) {
                    ++as_res;
                    other = other || !plain || st.g.N != emb.depth || st.g.ldr != emb.depth;
                }
            } else
                other = other || st.a == x0 || st.b == x0 || st.proj_residual == x0;
        }
        if (!other && as_x + as_res > 0) {
            for (size_t i = 1; i < s->steps.size(); ++i) {
                auto& st = s->steps[i];
                if (st.kind != fdx_session::Step::Gemm || (st.g.X != x0 && st.g.residual != x0))
                    continue;
                st.g.emb_a = emb.a;
                st.g.emb_a_rows = emb.g.M;
                st.g.emb_b = emb.b;
                st.g.emb_b_rows = emb.g.N;
                st.g.emb_err = m.err_flag;
                st.g.emb_x = st.g.X == x0;
                st.g.emb_res = st.g.residual == x0;
                if (st.g.emb_res)
                    st.g.residual = nullptr;
            }
            s->steps.erase(s->steps.begin());
        }
    }
    return set_int_launch(s->len_dev, 0) == FDX_OK;
}

// whether a greedy loop can let the last launch of a step embed the picked tokens for the next one: the step opens with
// the token + position embedding and ends in the per-workgroup maxima of the head
bool glue_mergeable(const fdx_session* s)
{
    static const bool on = [] { const char* e = std::getenv("FDX_DECODE_MERGE_GLUE"); return !(e && e[0] == '0'); }();
    return on && s->amax_part_count > 0 && !s->steps.empty() && s->steps[0].kind == fdx_session::Step::EmbedAdd && s->steps[0].depth % 4 == 0
        && s->history;
}

// enqueues the fused launches of one decode step; ids_dev [batch] floats, greedy ids go to next_dev.  merged: the step's
// embedding is already in place (the previous step's last launch, or the loop's prologue, put it there) and this step's
// last launch embeds the ids it picks.
fdx_status launch_steps(fdx_session* s, const float* ids_dev, float* next_dev, bool merged = false)
{
    fdx_model& m = *s->m;
    const int B = s->batch;
    fdx_status st = FDX_OK;
    for (size_t si = merged ? 1 : 0; si < s->steps.size(); ++si) {
        const auto& step = s->steps[si];
        const Op& o = m.ops[step.op];
        const fdx_act act = to_c(o.act);
        const fdx_act* actp = o.act.kind == FDX_ACT_NONE ? nullptr : &act;
        switch (step.kind) {
        case fdx_session::Step::EmbedAdd:
            st = embed_add_launch(ids_dev, B, step.a, step.g.M, step.b, step.g.N, s->len_dev, step.depth, step.out, m.err_flag, s->amax);
            break;
        case fdx_session::Step::Gemm:
            if (step.g.emb_x || step.g.emb_res) { // the ids of this call
                SkinnyParams g = step.g;
                g.emb_ids = ids_dev;
                st = skinny_gemm_launch(g);
            } else
                st = skinny_gemm_launch(step.g);
            break;
        case fdx_session::Step::Attn:
            st = mha_decode_dyn_launch(step.a, (int64_t)o.heads * o.dk, s->kc[step.op], s->vc[step.op], step.out, B, o.heads, o.dk, o.dv,
                s->len_dev, s->max_len, s->len + 1);
            break;
        case fdx_session::Step::AttnProj: {
            const Op& mo = m.ops[step.mha_op];
            st = mha_decode_proj_launch(step.a, (int64_t)mo.heads * mo.dk, s->kc[step.mha_op], s->vc[step.mha_op], B, mo.heads, s->len_dev,
                s->max_len, step.proj_w, step.proj_bias, step.proj_residual, step.depth, step.proj_act, step.depth, s->splitk_ws,
                fdx_session::kWsFloats, s->splitk_tickets, fdx_session::kTickets, step.out, s->len + 1);
            break;
        }
        case fdx_session::Step::LayerNorm:
            st = fdx_layernorm_f32(step.a, B, step.depth, o.dw[0], o.dw[1], o.eps, step.out);
            break;
        case fdx_session::Step::Add:
            st = fdx_eltwise_add_f32(step.a, step.b, (size_t)B * step.depth, (size_t)B * step.depth, actp, step.out);
            break;
        case fdx_session::Step::Act:
            st = fdx_activation_f32(step.a, (size_t)B * step.depth, actp, step.out);
            break;
        case fdx_session::Step::Softmax:
            st = fdx_softmax_f32(step.a, B, step.depth, 0, 0, step.out);
            break;
        }
        if (st != FDX_OK)
            return st;
    }
    // greedy ids (first maximum wins); the same launch records them by position and advances the cached
    // length on the device
    if (merged) {
        const auto& e = s->steps[0];
        return argmax_parts_embed_launch(s->amax_parts, s->amax_part_count, B, next_dev, s->len_dev, s->history, e.a, e.g.M, e.b, e.g.N, e.depth,
            e.out, m.err_flag);
    }
    if (s->amax_part_count > 0)
        return argmax_parts_launch(s->amax_parts, s->amax_part_count, B, next_dev, s->len_dev, s->history);
    return argmax_bump_launch(s->logits_buf, B, s->vocab, next_dev, s->len_dev, s->amax, s->history);
}

// one decode step, eager launches
fdx_status run_fast(fdx_session* s, const float* ids_dev, float* logits_dev, float* next_ids_dev)
{
    fdx_model& m = *s->m;
    FDX_REQUIRE(ids_dev, "session: null ids");
    FDX_REQUIRE(s->len + 1 <= s->max_len, "session: sequence length %d exceeds max_len %d", s->len + 1, s->max_len);
    std::lock_guard<std::mutex> lock(m.mu);
    fdx_status st = launch_steps(s, ids_dev, next_ids_dev ? next_ids_dev : s->ids_buf);
    if (st != FDX_OK)
        return st;
    if (logits_dev)
        FDX_HIP(hipMemcpyAsync(logits_dev, s->logits_buf, sizeof(float) * (size_t)s->batch * s->vocab, hipMemcpyDeviceToDevice, stream()));
    s->len += 1;
    return FDX_OK;
}

// `steps` greedy steps as replays of one captured step graph: the step reads its ids from ids_buf and
// writes the next ids back there, the visible length lives in device memory, so every replay launches
// the identical kernel sequence.  Ids are collected from the per-position history afterwards.
fdx_status run_fast_greedy(fdx_session* s, const float* first_ids_dev, int steps, float* tokens_dev, float* last_logits_dev)
{
    fdx_model& m = *s->m;
    FDX_REQUIRE(s->len + steps <= s->max_len, "session: sequence length %d exceeds max_len %d", s->len + steps, s->max_len);
    std::lock_guard<std::mutex> lock(m.mu);
    const int B = s->batch;
    hipStream_t st = stream();
    FDX_HIP(hipMemcpyAsync(s->ids_buf, first_ids_dev, sizeof(float) * B, hipMemcpyDeviceToDevice, st));
    // Where the step opens with the embedding launch and ends in the head's maxima, the replayed graph leaves the embedding
    // out: the loop's first one runs here, every later one rides in the last launch of the step before (63 -> 62 launches
    // per step on the GPT-2 shape).
    // (not where the loop would run past the position table: those steps keep the stand-alone embedding launch)
    const bool merged = glue_mergeable(s) && s->len + steps <= s->steps[0].g.N;
    if (merged) {
        const auto& e = s->steps[0];
        const fdx_status es = embed_add_launch(s->ids_buf, B, e.a, e.g.M, e.b, e.g.N, s->len_dev, e.depth, e.out, m.err_flag, s->amax);
        if (es != FDX_OK)
            return es;
    }
    hipGraphExec_t& step_graph = merged ? s->step_graph_merged : s->step_graph;
    if (!step_graph) {
        hipGraph_t graph = nullptr;
        FDX_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
        const fdx_status ls = launch_steps(s, s->ids_buf, s->ids_buf, merged);
        const hipError_t ce = hipStreamEndCapture(st, &graph);
        if (ls != FDX_OK) {
            if (graph)
                (void)hipGraphDestroy(graph);
            return ls;
        }
        FDX_HIP(ce);
        const hipError_t ie = hipGraphInstantiate(&step_graph, graph, nullptr, nullptr, 0);
        (void)hipGraphDestroy(graph);
        FDX_HIP(ie);
    }
    const int start = s->len;
    for (int i = 0; i < steps; ++i)
        FDX_HIP(hipGraphLaunch(step_graph, st));
    s->len += steps;
    FDX_HIP(hipMemcpyAsync(tokens_dev, s->history + (size_t)start * B, sizeof(float) * (size_t)steps * B, hipMemcpyDeviceToDevice, st));
    if (last_logits_dev)
        FDX_HIP(hipMemcpyAsync(last_logits_dev, s->logits_buf, sizeof(float) * (size_t)B * s->vocab, hipMemcpyDeviceToDevice, st));
    return FDX_OK;
}

} // namespace

extern "C" fdx_status fdx_session_create(fdx_model* m, int batch, int max_len, fdx_session** out)
{
    FDX_REQUIRE(m && out && batch > 0 && max_len > 0, "session_create: bad arguments");
    *out = nullptr;
    FDX_REQUIRE(m->inputs.size() == 2 && m->outputs.size() == 1,
        "session_create: a decoder model takes (ids, positions) and returns logits");
    FDX_REQUIRE(m->in_decl[0].size() == 1 && m->in_decl[1].size() == 1, "session_create: ids and positions must be rank-1 inputs");
    std::unique_ptr<fdx_session> s(new fdx_session);
    s->m = m;
    s->batch = batch;
    s->max_len = max_len;
    s->order = topo_order(*m);
    for (size_t p = 0; p < s->order.size(); ++p) {
        const Op& o = m->ops[s->order[p]];
        if (o.dead)
            continue;
        // layer variants the cached step does not implement
        if ((o.kind == OpKind::LayerNorm && o.rms) || (o.kind == OpKind::Add && (o.combine != FDX_COMBINE_ADD || o.scale != 1.0f))
            || (o.kind == OpKind::Softmax && o.log_after) || (o.kind == OpKind::MHA && o.gate)
            || (o.kind == OpKind::Act && !(o.act.kind == FDX_ACT_RELU || o.act.kind == FDX_ACT_GELU || o.act.kind == FDX_ACT_NONE))) {
            set_error("session_create: layer %s (%s) is not supported inside a decode session", o.name.c_str(), o.cls.c_str());
            return FDX_ERR_UNSUPPORTED;
        }
        switch (o.kind) {
        case OpKind::LayerNorm: {
            // a position is one (1, depth) row of the (T, depth) sample: only statistics over the depth axis keep
            // positions apart (layers/layer_normalization_layer.hpp:37-63 takes any axis set)
            const bool last_only = o.target_shape.size() == 1 && (o.target_shape[0] == -1 || o.target_shape[0] == 2);
            if (!last_only) {
                set_error("session_create: %s normalises over an axis other than the last; its statistics would mix positions",
                    o.name.c_str());
                return FDX_ERR_UNSUPPORTED;
            }
            break;
        }
        case OpKind::View:
            // Flatten / Reshape regroup the (T, depth) sample across positions; identity layers carry neither attribute
            if (o.flatten || !o.target_shape.empty()) {
                set_error("session_create: %s (%s) reshapes across positions", o.name.c_str(), o.cls.c_str());
                return FDX_ERR_UNSUPPORTED;
            }
            break;
        case OpKind::Input: case OpKind::Embedding: case OpKind::Add: case OpKind::Act:
        case OpKind::Softmax: case OpKind::Dense: // softmax runs along depth only (tensor.hpp:1165-1192)
            break;
        case OpKind::MHA: {
            const bool self = o.in[0] == o.in[1] && (o.in.size() == 2 || o.in[2] == o.in[0]);
            if (!self) {
                set_error("session_create: %s is not self-attention (query, value and key must be the same tensor)", o.name.c_str());
                return FDX_ERR_UNSUPPORTED;
            }
            s->last_mha_pos = (int)p;
            float *k = nullptr, *v = nullptr;
            FDX_HIP(hipMalloc(&k, sizeof(float) * (size_t)batch * max_len * o.heads * o.dk));
            s->kc[s->order[p]] = k;
            FDX_HIP(hipMalloc(&v, sizeof(float) * (size_t)batch * max_len * o.heads * o.dv));
            s->vc[s->order[p]] = v;
            break;
        }
        default:
            set_error("session_create: layer %s (%s) mixes positions; only per-position layers and self-attention can be cached",
                o.name.c_str(), o.cls.c_str());
            return FDX_ERR_UNSUPPORTED;
        }
    }
    std::vector<int> memo(m->ops.size(), -1);
    s->vocab = depth_of(*m, m->outputs[0], memo);
    s->fast = build_fast_plan(s.get());
    if (!s->fast)
        s->steps.clear();
    *out = s.release();
    return FDX_OK;
}

extern "C" fdx_status fdx_session_destroy(fdx_session* s)
{
    delete s;
    return FDX_OK;
}

extern "C" fdx_status fdx_session_reset(fdx_session* s)
{
    FDX_REQUIRE(s, "session_reset: null session");
    s->len = 0;
    if (s->len_dev)
        return set_int_launch(s->len_dev, 0);
    return FDX_OK;
}

extern "C" fdx_status fdx_session_length(const fdx_session* s, int* len)
{
    FDX_REQUIRE(s && len, "session_length: null argument");
    *len = s->len;
    return FDX_OK;
}

extern "C" fdx_status fdx_session_prefill(fdx_session* s, const float* ids_dev, int t, float* logits_dev, float* next_ids_dev)
{
    FDX_REQUIRE(s, "session_prefill: null session");
    fdx_status st = run(s, ids_dev, t, logits_dev, next_ids_dev);
    if (st == FDX_OK && s->len_dev)
        st = set_int_launch(s->len_dev, s->len);
    return st;
}

extern "C" fdx_status fdx_session_decode_step(fdx_session* s, const float* ids_dev, float* logits_dev, float* next_ids_dev)
{
    FDX_REQUIRE(s, "session_decode_step: null session");
    if (s->fast)
        return run_fast(s, ids_dev, logits_dev, next_ids_dev);
    return run(s, ids_dev, 1, logits_dev, next_ids_dev);
}

extern "C" fdx_status fdx_session_decode_greedy(fdx_session* s, const float* first_ids_dev, int steps, float* tokens_dev,
    float* last_logits_dev)
{
    FDX_REQUIRE(s && first_ids_dev && tokens_dev && steps > 0, "session_decode_greedy: bad arguments");
    // FDX_DECODE_GRAPH=0 keeps the eager launches (tools that intercept HIP calls may not cope with graphs)
    static const bool use_graph = [] {
        const char* e = std::getenv("FDX_DECODE_GRAPH");
        return !(e && e[0] == '0');
    }();
    if (s->fast && use_graph && !profiling())
        return run_fast_greedy(s, first_ids_dev, steps, tokens_dev, last_logits_dev);
    for (int i = 0; i < steps; ++i) {
        const float* ids = i == 0 ? first_ids_dev : tokens_dev + (size_t)(i - 1) * s->batch;
        float* logits = i + 1 == steps ? last_logits_dev : nullptr;
        float* next = tokens_dev + (size_t)i * s->batch;
        fdx_status st = s->fast ? run_fast(s, ids, logits, next) : run(s, ids, 1, logits, next);
        if (st != FDX_OK)
            return st;
    }
    return FDX_OK;
}

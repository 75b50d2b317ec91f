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
#include <map>

#include "model.hpp"

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
                st = fdx_gemm_bias_act_f32(merged, nv, o.dw[6], nv, (int)R, o.dout, (int)nv, 1.f, o.dw[7], 0, nullptr, nullptr, out, o.dout,
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
        switch (o.kind) {
        case OpKind::Input: case OpKind::Embedding: case OpKind::Add: case OpKind::LayerNorm: case OpKind::Act:
        case OpKind::Softmax: case OpKind::Dense: case OpKind::View:
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
    return run(s, ids_dev, t, logits_dev, next_ids_dev);
}

extern "C" fdx_status fdx_session_decode_step(fdx_session* s, const float* ids_dev, float* logits_dev, float* next_ids_dev)
{
    FDX_REQUIRE(s, "session_decode_step: null session");
    return run(s, ids_dev, 1, logits_dev, next_ids_dev);
}

extern "C" fdx_status fdx_session_decode_greedy(fdx_session* s, const float* first_ids_dev, int steps, float* tokens_dev,
    float* last_logits_dev)
{
    FDX_REQUIRE(s && first_ids_dev && tokens_dev && steps > 0, "session_decode_greedy: bad arguments");
    for (int i = 0; i < steps; ++i) {
        const float* ids = i == 0 ? first_ids_dev : tokens_dev + (size_t)(i - 1) * s->batch;
        fdx_status st = run(s, ids, 1, i + 1 == steps ? last_logits_dev : nullptr, tokens_dev + (size_t)i * s->batch);
        if (st != FDX_OK)
            return st;
    }
    return FDX_OK;
}

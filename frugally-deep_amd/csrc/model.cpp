// Loader, load-time fusion, launch planner and executor behind fdx_model_*.
//
// Reads the converted-JSON format that frugally-deep's read_model consumes
// (include/fdeep/model.hpp:198-281, include/fdeep/import_model.hpp), turns the layer graph
// into a flat op list, fuses what the GPU can do in one pass (BatchNormalization into the
// preceding convolution's weights, ReLU/GELU and residual Add into GEMM epilogues,
// ZeroPadding2D into the consumer's padding predicate), uploads the weights once, and runs
// `batch` independent samples per launch with the batch as the outermost axis.
#include "model.hpp"

#include <algorithm>
#include <map>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <condition_variable>
#include <set>
#include <thread>
#include <tuple>

#include "einsum.hpp"
#include "igemm_params.hpp"
#include "json.hpp"

using namespace fdx;
using json::Value;

namespace fdx {

Plan::~Plan()
{
    for (auto& b : blocks)
        if (b.p)
            (void)hipFree(b.p);
}

float* plan_alloc(Plan& p, size_t bytes, int* block_index)
{
    bytes = (bytes + 255) & ~(size_t)255;
    int best = -1;
    for (size_t i = 0; i < p.blocks.size(); ++i)
        if (!p.blocks[i].busy && p.blocks[i].bytes >= bytes && (best < 0 || p.blocks[i].bytes < p.blocks[best].bytes))
            best = (int)i;
    if (best < 0) {
        Block b;
        if (hipMalloc(&b.p, bytes) != hipSuccess)
            return nullptr;
        b.bytes = bytes;
        p.blocks.push_back(b);
        best = (int)p.blocks.size() - 1;
    }
    p.blocks[best].busy = true;
    *block_index = best;
    return static_cast<float*>(p.blocks[best].p);
}

namespace {

    struct FormatError : std::runtime_error {
        using std::runtime_error::runtime_error;
    };
    struct Unsupported : std::runtime_error {
        using std::runtime_error::runtime_error;
    };

    // include/fdeep/import_model.hpp:274-297
    std::vector<float> decode_floats(const Value& v)
    {
        if (!(v.is_array() || v.is_string()))
            throw FormatError("invalid float array format");
        std::vector<float> out;
        if (v.is_array() && v.size() > 0 && v.arr[0].is_number()) {
            out.reserve(v.size());
            for (const auto& e : v.arr)
                out.push_back((float)e.number());
            return out;
        }
        std::vector<uint8_t> bytes;
        auto feed = [&](const Value& s) {
            if (!s.is_string() || !base64_decode_append(s.s, s.slen, bytes))
                throw FormatError("invalid base64 float data");
        };
        if (v.is_string())
            feed(v);
        else {
            size_t chars = 0;
            for (const auto& e : v.arr)
                chars += e.is_string() ? e.slen : 0;
            bytes.reserve(chars / 4 * 3 + 8);
            for (const auto& e : v.arr)
                feed(e);
        }
        if (bytes.size() % 4 != 0)
            throw FormatError("invalid float vector data");
        out.resize(bytes.size() / 4);
        if (!bytes.empty()) // an empty array has no buffer to copy from
            std::memcpy(out.data(), bytes.data(), bytes.size());
        return out;
    }

    struct Conn {
        std::string layer;
        int node, tensor;
    };

    // import_model.hpp:323-372
    Conn conn_from_triple(const Value& v)
    {
        if (!v.is_array() || v.size() < 3)
            throw FormatError("invalid format for inbound node");
        return { v.at((size_t)0).str(), (int)v.at(1).integer(), (int)v.at(2).integer() };
    }
    std::vector<Conn> model_connections(const Value& v)
    {
        if (!v.is_array())
            throw FormatError("input_layers/output_layers must be an array");
        std::vector<Conn> r;
        if (v.size() > 0 && !v.arr[0].is_array()) {
            r.push_back(conn_from_triple(v));
            return r;
        }
        for (const auto& e : v.arr)
            r.push_back(conn_from_triple(e));
        return r;
    }
    Conn conn_from_arg(const Value& a)
    {
        const Value* cfg = a.is_object() ? a.find("config") : nullptr;
        const Value* kh = cfg ? cfg->find("keras_history") : nullptr;
        if (!kh)
            throw FormatError("No keras_history on node connection. Constant-value tensors are not supported.");
        return conn_from_triple(*kh);
    }
    std::vector<std::vector<Conn>> inbound_nodes(const Value& layer)
    {
        std::vector<std::vector<Conn>> nodes;
        const Value* in = layer.find("inbound_nodes");
        if (!in || !in->is_array())
            throw FormatError("no inbound nodes");
        for (const auto& n : in->arr) {
            const Value& args = n.at("args");
            if (!args.is_array())
                throw FormatError("node args need to be an array");
            std::vector<Conn> c;
            if (args.size() > 0 && args.arr[0].is_array()) {
                if (args.size() != 1)
                    throw FormatError("invalid args format");
                for (const auto& a : args.arr[0].arr)
                    c.push_back(conn_from_arg(a));
            } else {
                for (const auto& a : args.arr)
                    c.push_back(conn_from_arg(a));
            }
            nodes.push_back(std::move(c));
        }
        return nodes;
    }

    int padding_from(const std::string& s)
    {
        if (s == "valid") return 0;
        if (s == "same") return 1;
        if (s == "causal") return 2;
        throw FormatError("no padding");
    }
    void pair_from(const Value& v, int& a, int& b)
    {
        if (v.is_array() && v.size() == 2) {
            a = (int)v.at((size_t)0).integer();
            b = (int)v.at(1).integer();
        } else if (v.is_array() && v.size() == 1) { // 1-D layers: width only
            a = 1;
            b = (int)v.at((size_t)0).integer();
        } else { // a bare number is a width (create_shape2, import_model.hpp:229-242)
            a = 1;
            b = (int)v.integer();
        }
    }

    // Layer class names that are the identity at inference (import_model.hpp:1796-1838)
    const std::set<std::string> kIdentity = { "Identity", "Dropout", "Masking", "ActivityRegularization", "AlphaDropout",
        "FixedDropout", "SpatialDropout1D", "SpatialDropout2D", "SpatialDropout3D", "GaussianDropout", "GaussianNoise",
        "RandomBrightness", "RandomContrast", "RandomCrop", "RandomFlip", "RandomHeight", "RandomRotation",
        "RandomTranslation", "RandomWidth", "RandomZoom", "RandomColorDegeneration", "RandomColorJitter", "RandomElasticTransform", "RandomErasing", "RandomGaussianBlur",
        "RandomGrayscale", "RandomHue", "RandomInvert", "RandomPerspective", "RandomPosterization", "RandomSaturation",
        "RandomSharpness", "RandomShear", "AugMix", "CutMix", "Equalization", "MaxNumBoundingBoxes", "MixUp", "Pipeline",
        "RandAugment", "Solarization" };

    // Sets an activation by name; returns false for "softmax" (caller schedules the softmax kernel).
    // import_model.hpp:1649-1700; relu parameters only when max_value is present and non-null (:1289-1302).
    enum class ActParse { Epilogue, Softmax, Linear, Standalone, LogSoftmax };
    float cfg_float(const Value* cfg, const char* key, float dflt)
    {
        const Value* v = cfg ? cfg->find(key) : nullptr;
        return v && v->is_number() ? (float)v->number() : dflt;
    }
    // import_model.hpp:1649-1700 (names), :1200-1385 (parameters and their defaults)
    ActParse parse_activation(const std::string& type, const Value* cfg, Act& act)
    {
        const float big = 3.402823466e+38f;
        auto plain = [&](int kind) {
            act = { kind, big, 0.f, 0.f };
            return ActParse::Standalone;
        };
        if (type == "linear")
            return ActParse::Linear;
        if (type == "softmax")
            return ActParse::Softmax;
        if (type == "log_softmax")
            return ActParse::LogSoftmax;
        if (type == "relu") {
            act = { FDX_ACT_RELU, big, 0.f, 0.f };
            const Value* mv = cfg ? cfg->find("max_value") : nullptr;
            if (mv && !mv->is_null()) { // parameters only when max_value is present and non-null (:1289-1302)
                act.max_value = (float)mv->number();
                act.negative_slope = (float)cfg->at("negative_slope").number();
                act.threshold = (float)cfg->at("threshold").number();
            }
            return ActParse::Epilogue;
        }
        if (type == "relu6") {
            act = { FDX_ACT_RELU, 6.f, 0.f, 0.f };
            return ActParse::Epilogue;
        }
        if (type == "gelu") {
            const Value* ap = cfg ? cfg->find("approximate") : nullptr;
            if (ap && !ap->is_null() && ap->boolean())
                throw FormatError("Gelu with approximate = True is not supported.");
            act = { FDX_ACT_GELU, big, 0.f, 0.f };
            return ActParse::Epilogue;
        }
        if (type == "tanh") return plain(FDX_ACT_TANH);
        if (type == "sigmoid") return plain(FDX_ACT_SIGMOID);
        if (type == "swish" || type == "silu") return plain(FDX_ACT_SWISH);
        if (type == "hard_sigmoid") return plain(FDX_ACT_HARD_SIGMOID);
        if (type == "selu") return plain(FDX_ACT_SELU);
        if (type == "exponential") return plain(FDX_ACT_EXPONENTIAL);
        if (type == "softsign") return plain(FDX_ACT_SOFTSIGN);
        if (type == "softplus") return plain(FDX_ACT_SOFTPLUS);
        if (type == "sparse_plus") return plain(FDX_ACT_SPARSE_PLUS);
        if (type == "tanh_shrink") return plain(FDX_ACT_TANH_SHRINK);
        if (type == "log_sigmoid") return plain(FDX_ACT_LOG_SIGMOID);
        if (type == "hard_tanh") return plain(FDX_ACT_HARD_TANH);
        if (type == "elu" || type == "celu") {
            act = { FDX_ACT_ELU, big, cfg_float(cfg, "alpha", 1.0f), 0.f };
            return ActParse::Standalone;
        }
        if (type == "leaky_relu") {
            act = { FDX_ACT_LEAKY_RELU, big, cfg_float(cfg, "negative_slope", 0.2f), 0.f };
            return ActParse::Standalone;
        }
        if (type == "hard_shrink" || type == "soft_shrink") {
            if (!cfg || !cfg->find("threshold"))
                throw FormatError(type + " needs a threshold");
            act = { type[0] == 'h' ? FDX_ACT_HARD_SHRINK : FDX_ACT_SOFT_SHRINK, big, 0.f, (float)cfg->at("threshold").number() };
            return ActParse::Standalone;
        }
        if (type == "squareplus") {
            act = { FDX_ACT_SQUARE_PLUS, cfg_float(cfg, "b", 4.0f), 0.f, 0.f };
            return ActParse::Standalone;
        }
        if (type == "threshold") { // Keras renamed threshold_value -> threshold, value -> default_value (:1277-1287)
            const float thr = cfg && cfg->find("threshold") ? cfg_float(cfg, "threshold", 0.f) : cfg_float(cfg, "threshold_value", 0.f);
            const float dv = cfg && cfg->find("default_value") ? cfg_float(cfg, "default_value", 0.f) : cfg_float(cfg, "value", 0.f);
            act = { FDX_ACT_THRESHOLD, dv, 0.f, thr };
            return ActParse::Standalone;
        }
        throw Unsupported("unknown activation type: " + type);
    }

    // layer classes that are one element-wise activation (import_model.hpp:1839-1865)
    const std::map<std::string, std::string> kActivationLayers = { { "LeakyReLU", "leaky_relu" }, { "LeakyRelu", "leaky_relu" },
        { "ELU", "elu" }, { "Elu", "elu" }, { "Celu", "celu" }, { "ReLU", "relu" }, { "Relu6", "relu6" }, { "Exp", "exponential" },
        { "Gelu", "gelu" }, { "Selu", "selu" }, { "Silu", "silu" }, { "Tanh", "tanh" }, { "TanhShrink", "tanh_shrink" },
        { "Threshold", "threshold" }, { "Sigmoid", "sigmoid" }, { "HardShrink", "hard_shrink" }, { "HardSigmoid", "hard_sigmoid" },
        { "HardTanh", "hard_tanh" }, { "SoftShrink", "soft_shrink" }, { "Softplus", "softplus" }, { "Softsign", "softsign" },
        { "SparsePlus", "sparse_plus" }, { "Squareplus", "squareplus" }, { "LogSigmoid", "log_sigmoid" }, { "LogSoftmax", "log_softmax" },
        { "Softmax", "softmax" } };

    // One level of the layer graph: the top-level model or one application of a nested
    // Functional model (create_model_layer, import_model.hpp:397-424).  A nested level reads its
    // parameters under "<outer names>_<layer>" and its InputLayers are bound to the outer operands.
    struct Scope {
        std::map<std::string, const Value*> layers;
        std::string prefix;
        std::map<std::string, int> input_ops;
        std::map<std::tuple<std::string, int, int>, int> memo;
        std::set<std::tuple<std::string, int, int>> building; // connections whose producers are being resolved right now
    };

    struct Builder {
        fdx_model& m;
        const Value& params;
        std::vector<std::unique_ptr<Scope>> scopes;
        const fdx_custom_layer* customs = nullptr;
        int n_customs = 0;

        // trainable_params lookup handed to a custom layer's factory; the decoded vectors live until it returns
        struct ParamCtx {
            Builder* b;
            const Scope* sc;
            std::vector<std::vector<float>> keep;
        };
        static fdx_status get_param_cb(void* ctx, const char* layer, const char* key, const float** values, size_t* count)
        {
            auto* pc = static_cast<ParamCtx*>(ctx);
            try {
                pc->keep.push_back(decode_floats(pc->b->param(*pc->sc, layer, key)));
            } catch (const std::exception& e) {
                set_error("%s", e.what());
                return FDX_ERR_FORMAT;
            }
            if (values)
                *values = pc->keep.back().data();
            if (count)
                *count = pc->keep.back().size();
            return FDX_OK;
        }

        const Value& param(const Scope& sc, const std::string& layer, const char* key)
        {
            const std::string full = sc.prefix + layer;
            const Value* l = params.find(full.c_str());
            if (!l)
                throw FormatError("missing trainable_params for layer " + full);
            return l->at(key);
        }

        static void index_layers(Scope& sc, const Value& layers)
        {
            if (!layers.is_array())
                throw FormatError("missing layers array");
            for (const auto& l : layers.arr) {
                const std::string name = l.at("name").str();
                if (sc.layers.count(name))
                    throw FormatError("layer names must be unique");
                sc.layers[name] = &l;
            }
        }

        int add_op(Op&& op)
        {
            m.ops.push_back(std::move(op));
            return (int)m.ops.size() - 1;
        }

        // an element-wise activation (or softmax / log_softmax) as an op of its own after `in`
        int activation_op(const std::string& name, const std::string& type, const Value* cfg, int in)
        {
            Op op;
            op.name = name;
            op.cls = "Activation";
            op.in = { in };
            switch (parse_activation(type, cfg, op.act)) {
            case ActParse::Linear: op.kind = OpKind::View; break;
            case ActParse::Softmax: op.kind = OpKind::Softmax; break;
            case ActParse::LogSoftmax: op.kind = OpKind::Softmax; op.log_after = true; break;
            case ActParse::Epilogue:
            case ActParse::Standalone: op.kind = OpKind::Act; break;
            }
            return add_op(std::move(op));
        }

        // applies config["activation"] after the op (import_model.hpp:1953-1962): ReLU / GELU ride in the producer's
        // epilogue, softmax is flagged on the producer, everything else becomes an activation op of its own
        int with_fused_activation(int idx, const Value& cfg)
        {
            const Value* a = cfg.find("activation");
            if (!a)
                return idx;
            if (!a->is_string())
                throw FormatError("Layer activation must be a string.");
            Act act = m.ops[idx].act;
            switch (parse_activation(a->str(), nullptr, act)) {
            case ActParse::Linear: return idx;
            case ActParse::Softmax: m.ops[idx].softmax = true; return idx;
            case ActParse::Epilogue: m.ops[idx].act = act; return idx;
            case ActParse::Standalone:
            case ActParse::LogSoftmax: return activation_op(m.ops[idx].name + "_activation", a->str(), nullptr, idx);
            }
            return idx;
        }

        int build(Scope& sc, const Conn& c)
        {
            auto key = std::make_tuple(c.layer, c.node, c.tensor);
            auto& memo = sc.memo;
            auto it = memo.find(key);
            if (it != memo.end())
                return it->second;
            auto lit = sc.layers.find(c.layer);
            if (lit == sc.layers.end())
                throw FormatError("dangling connection to layer " + c.layer);
            // a layer that (directly or through others) names itself as its input would recurse without end
            if (!sc.building.insert(key).second)
                throw FormatError("cyclic connection at layer " + c.layer);
            struct Leave {
                std::set<std::tuple<std::string, int, int>>& s;
                std::tuple<std::string, int, int> k;
                ~Leave() { s.erase(k); }
            } leave { sc.building, key };
            const Value& L = *lit->second;
            const std::string cls = L.at("class_name").str();
            const Value& cfg = L.at("config");
            if (cls == "InputLayer") {
                auto io = sc.input_ops.find(c.layer);
                if (io == sc.input_ops.end())
                    throw FormatError("input layer " + c.layer + " is not listed in input_layers");
                return memo[key] = io->second;
            }
            const bool nested = cls == "Functional" || cls == "Model";
            if (c.tensor != 0 && !nested)
                throw Unsupported("layers with several output tensors are not supported: " + c.layer);
            auto nodes = inbound_nodes(L);
            // a nested model counts its own construction as node 0 (layers/model_layer.hpp:36-44)
            const int node = nested && c.node >= 1 ? c.node - 1 : c.node;
            if (node < 0 || node >= (int)nodes.size())
                throw FormatError("invalid node index for layer " + c.layer);
            std::vector<int> ins;
            for (const auto& ic : nodes[node])
                ins.push_back(build(sc, ic));
            if (ins.empty())
                throw FormatError("layer without inputs: " + c.layer);
            if (nested) {
                scopes.emplace_back(new Scope);
                Scope& inner = *scopes.back();
                inner.prefix = sc.prefix + c.layer + "_";
                index_layers(inner, cfg.at("layers"));
                const auto inner_in = model_connections(cfg.at("input_layers"));
                const auto inner_out = model_connections(cfg.at("output_layers"));
                if (inner_in.size() != ins.size())
                    throw FormatError("invalid number of input tensors for this model: " + std::to_string(inner_in.size())
                        + " required but " + std::to_string(ins.size()) + " provided");
                for (size_t i = 0; i < ins.size(); ++i)
                    inner.input_ops[inner_in[i].layer] = ins[i];
                if (c.tensor < 0 || c.tensor >= (int)inner_out.size())
                    throw FormatError("invalid tensor index for nested model " + c.layer);
                // every output of this application is built now so they share the inner operands
                int chosen = -1;
                for (size_t t = 0; t < inner_out.size(); ++t) {
                    const int r = build(inner, inner_out[t]);
                    sc.memo[std::make_tuple(c.layer, c.node, (int)t)] = r;
                    if ((int)t == c.tensor)
                        chosen = r;
                }
                return chosen;
            }

            Op op;
            op.name = sc.prefix + c.layer;
            op.cls = cls;
            op.in = ins;
            int result;
            const fdx_custom_layer* custom = nullptr;
            for (int i = 0; i < n_customs && !custom; ++i)
                if (customs[i].class_name && cls == customs[i].class_name)
                    custom = &customs[i];
            if (custom) {
                // a registered class takes precedence over a built-in one (import_model.hpp:1944-1950)
                if (!custom->create || !custom->apply)
                    throw FormatError("custom layer " + cls + " lacks create / apply");
                op.kind = OpKind::Host;
                fdx_host_layer hl;
                hl.vt = *custom;
                ParamCtx pc { this, &sc, {} };
                if (custom->create(custom->user, c.layer.c_str(), L.s, L.slen, &Builder::get_param_cb, &pc, &hl.instance) != FDX_OK)
                    throw FormatError("custom layer " + c.layer + " could not be created: " + fdx_last_error());
                m.host_layers.push_back(hl);
                op.host_index = (int)m.host_layers.size() - 1;
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (kIdentity.count(cls)) {
                op.kind = OpKind::View;
                result = add_op(std::move(op));
            } else if (cls == "Conv2D" || cls == "Conv1D") {
                op.kind = OpKind::Conv2D;
                op.padding = padding_from(cfg.at("padding").str());
                pair_from(cfg.at("strides"), op.sy, op.sx);
                pair_from(cfg.at("dilation_rate"), op.dy, op.dx);
                pair_from(cfg.at("kernel_size"), op.kh, op.kw);
                op.cout = (int)cfg.at("filters").integer();
                op.hw.resize(2);
                op.hw[0] = decode_floats(param(sc, c.layer, "weights"));
                if (cfg.at("use_bias").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                else
                    op.hw[1].assign(op.cout, 0.f);
                if ((int)op.hw[1].size() != op.cout)
                    throw FormatError("size of bias does not match");
                if (op.hw[0].size() % ((size_t)op.kh * op.kw * op.cout) != 0)
                    throw FormatError("invalid number of weights");
                op.n_in = (int)(op.hw[0].size() / ((size_t)op.kh * op.kw * op.cout));
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "Conv2DTranspose" || cls == "Conv1DTranspose") {
                // convolve_transposed (convolution.hpp:443-469, import_model.hpp:528-556): zeros between the input pixels,
                // then a stride-1 convolution with the filter mirrored in height and width (filter.hpp:94-97). "valid"
                // pads the zero-stuffed image by the inflated filter size minus one on every side, which is an explicit
                // zero frame around a valid window; "same" is the ordinary stride-1 rule. "causal" cannot pass the
                // reference's own output-width assertion (convolution.hpp:243) and is refused at load.
                const int pad_mode = padding_from(cfg.at("padding").str());
                if (pad_mode == 2)
                    throw FormatError("output width does not match");
                int ry = 1, rx = 1;
                pair_from(cfg.at("strides"), ry, rx);
                if (ry != 1 || rx != 1) {
                    Op dil;
                    dil.kind = OpKind::Dilate;
                    dil.name = op.name + "_zero_insertion";
                    dil.cls = cls;
                    dil.in = ins;
                    dil.kh = ry;
                    dil.kw = rx;
                    dil.trailing = pad_mode == 1;
                    op.in = { add_op(std::move(dil)) };
                }
                op.kind = OpKind::Conv2D;
                op.padding = pad_mode;
                pair_from(cfg.at("dilation_rate"), op.dy, op.dx);
                pair_from(cfg.at("kernel_size"), op.kh, op.kw);
                op.cout = (int)cfg.at("filters").integer();
                op.hw.resize(2);
                std::vector<float> wj = decode_floats(param(sc, c.layer, "weights"));
                if (cfg.at("use_bias").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                else
                    op.hw[1].assign(op.cout, 0.f);
                if ((int)op.hw[1].size() != op.cout)
                    throw FormatError("size of bias does not match");
                if (wj.empty() || wj.size() % ((size_t)op.kh * op.kw * op.cout) != 0)
                    throw FormatError("invalid number of weights");
                op.n_in = (int)(wj.size() / ((size_t)op.kh * op.kw * op.cout));
                op.hw[0].resize(wj.size()); // [cout][kh][kw][cin], taps mirrored
                for (int n = 0; n < op.cout; ++n)
                    for (int y = 0; y < op.kh; ++y)
                        for (int x = 0; x < op.kw; ++x)
                            std::copy_n(&wj[(((size_t)n * op.kh + (op.kh - 1 - y)) * op.kw + (op.kw - 1 - x)) * op.n_in], op.n_in,
                                &op.hw[0][(((size_t)n * op.kh + y) * op.kw + x) * op.n_in]);
                if (pad_mode == 0) {
                    const int ekh = (op.kh - 1) * op.dy + 1, ekw = (op.kw - 1) * op.dx + 1;
                    op.zp[0] = op.zp[1] = ekh - 1;
                    op.zp[2] = op.zp[3] = ekw - 1;
                }
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "DepthwiseConv2D" || cls == "DepthwiseConv1D") {
                op.kind = OpKind::DWConv2D;
                op.padding = padding_from(cfg.at("padding").str());
                pair_from(cfg.at("strides"), op.sy, op.sx);
                pair_from(cfg.at("dilation_rate"), op.dy, op.dx);
                pair_from(cfg.at("kernel_size"), op.kh, op.kw);
                std::vector<float> sw = decode_floats(param(sc, c.layer, "slice_weights"));
                if (sw.size() % ((size_t)op.kh * op.kw) != 0)
                    throw FormatError("invalid number of weights");
                const int ch = (int)(sw.size() / ((size_t)op.kh * op.kw));
                op.cout = op.n_in = ch;
                op.hw.resize(2);
                op.hw[0].resize(sw.size()); // [c][kh][kw] -> [kh][kw][c]
                for (int z = 0; z < ch; ++z)
                    for (int t = 0; t < op.kh * op.kw; ++t)
                        op.hw[0][(size_t)t * ch + z] = sw[(size_t)z * op.kh * op.kw + t];
                if (cfg.at("use_bias").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                else
                    op.hw[1].assign(ch, 0.f);
                if ((int)op.hw[1].size() != ch)
                    throw FormatError("size of bias does not match");
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "Dense") {
                op.kind = OpKind::Dense;
                op.units = (int)cfg.at("units").integer();
                std::vector<float> w = decode_floats(param(sc, c.layer, "weights"));
                op.hw.resize(2);
                if (cfg.at("use_bias").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                else
                    op.hw[1].assign(op.units, 0.f);
                if ((int)op.hw[1].size() != op.units || op.units == 0 || w.size() % (size_t)op.units != 0)
                    throw FormatError("size of bias does not match");
                op.n_in = (int)(w.size() / (size_t)op.units);
                op.hw[0].resize(w.size()); // [in][out] -> [out][in]
                for (int i = 0; i < op.n_in; ++i)
                    for (int o = 0; o < op.units; ++o)
                        op.hw[0][(size_t)o * op.n_in + i] = w[(size_t)i * op.units + o];
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "BatchNormalization") {
                op.kind = OpKind::Affine;
                std::vector<float> mean = decode_floats(param(sc, c.layer, "moving_mean"));
                std::vector<float> var = decode_floats(param(sc, c.layer, "moving_variance"));
                std::vector<float> gamma, beta;
                if (cfg.at("scale").boolean())
                    gamma = decode_floats(param(sc, c.layer, "gamma"));
                if (cfg.at("center").boolean())
                    beta = decode_floats(param(sc, c.layer, "beta"));
                const Value& ax = cfg.at("axis");
                if (ax.is_array() && ax.size() != 1)
                    throw FormatError("invalid axis configuration");
                op.ln_axes = (int)(ax.is_array() ? ax.at((size_t)0).integer() : ax.integer()); // checked at plan time
                const float eps = (float)cfg.at("epsilon").number();
                if (var.size() != mean.size() || (!gamma.empty() && gamma.size() != mean.size())
                    || (!beta.empty() && beta.size() != mean.size()))
                    throw FormatError("invalid sizes");
                // tensor.hpp:773-793: inv = gamma / sqrt(var + eps); y = x * inv + (beta - mean * inv)
                op.hw.resize(2);
                op.hw[0].resize(mean.size());
                op.hw[1].resize(mean.size());
                for (size_t i = 0; i < mean.size(); ++i) {
                    const float inv = (1.0f / std::sqrt(var[i] + eps)) * (gamma.empty() ? 1.f : gamma[i]);
                    op.hw[0][i] = inv;
                    op.hw[1][i] = (beta.empty() ? 0.f : beta[i]) - mean[i] * inv;
                }
                op.cout = (int)mean.size();
                result = add_op(std::move(op));
            } else if (cls == "Rescaling") {
                // y = scale * x + offset with one pair for the whole tensor (layers/rescaling_layer.hpp:30-40)
                op.kind = OpKind::Affine;
                op.hw.resize(2);
                op.hw[0] = { (float)cfg.at("scale").number() };
                op.hw[1] = { (float)cfg.at("offset").number() };
                op.cout = 1;
                op.affine_scalar = true;
                result = add_op(std::move(op));
            } else if (cls == "Normalization") {
                // (x - mean) / max(sqrt(variance), 1e-7), or its inverse; one pair for the whole tensor or one per slice of
                // the given axis (layers/normalization_layer.hpp:36-75, import_model.hpp:1392-1404)
                op.kind = OpKind::Affine;
                const std::vector<float> mean = decode_floats(param(sc, c.layer, "mean"));
                const std::vector<float> var = decode_floats(param(sc, c.layer, "variance"));
                const Value& ax = cfg.at("axis");
                const size_t n_axes = ax.is_array() ? ax.size() : (ax.is_null() ? 0 : 1);
                if (n_axes > 1)
                    throw FormatError("Unsupported number of axes for Normalization layer");
                if (mean.size() != var.size() || var.empty() || (n_axes == 0 && var.size() != 1))
                    throw FormatError("Invalid number of variance values in Normalization layer.");
                const Value* inv = cfg.find("invert");
                const bool invert = inv && inv->boolean();
                op.hw.resize(2);
                op.hw[0].resize(var.size());
                op.hw[1].resize(var.size());
                for (size_t i = 0; i < var.size(); ++i) {
                    const float sd = std::fmax(std::sqrt(var[i]), 1e-7f);
                    op.hw[0][i] = invert ? sd : 1.0f / sd;
                    op.hw[1][i] = invert ? mean[i] : -mean[i] / sd;
                }
                op.cout = (int)var.size();
                op.affine_scalar = n_axes == 0;
                if (n_axes == 1)
                    op.ln_axes = (int)(ax.is_array() ? ax.at((size_t)0).integer() : ax.integer());
                result = add_op(std::move(op));
            } else if (cls == "SeparableConv2D" || cls == "SeparableConv1D") {
                // depthwise part without bias or activation, then a 1x1 valid convolution that carries the bias and the
                // layer's activation (layers/separable_conv_2d_layer.hpp:26-55, import_model.hpp:558-592)
                Op dw;
                dw.kind = OpKind::DWConv2D;
                dw.name = op.name + "_depthwise_part";
                dw.cls = cls;
                dw.in = ins;
                dw.padding = padding_from(cfg.at("padding").str());
                pair_from(cfg.at("strides"), dw.sy, dw.sx);
                pair_from(cfg.at("dilation_rate"), dw.dy, dw.dx);
                pair_from(cfg.at("kernel_size"), dw.kh, dw.kw);
                std::vector<float> sw = decode_floats(param(sc, c.layer, "slice_weights"));
                if (sw.size() % ((size_t)dw.kh * dw.kw) != 0)
                    throw FormatError("invalid number of weights");
                const int ch = (int)(sw.size() / ((size_t)dw.kh * dw.kw));
                dw.cout = dw.n_in = ch;
                dw.hw.resize(2);
                dw.hw[0].resize(sw.size()); // [c][kh][kw] -> [kh][kw][c]
                for (int z = 0; z < ch; ++z)
                    for (int t = 0; t < dw.kh * dw.kw; ++t)
                        dw.hw[0][(size_t)t * ch + z] = sw[(size_t)z * dw.kh * dw.kw + t];
                dw.hw[1].assign(ch, 0.f);
                const int dwi = add_op(std::move(dw));
                op.kind = OpKind::Conv2D;
                op.in = { dwi };
                op.cout = (int)cfg.at("filters").integer();
                op.n_in = ch;
                op.hw.resize(2);
                op.hw[0] = decode_floats(param(sc, c.layer, "stack_weights")); // [cout][1][1][cin]
                if (op.hw[0].size() != (size_t)op.cout * ch)
                    throw FormatError("invalid weights sizes");
                if (cfg.at("use_bias").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                else
                    op.hw[1].assign(op.cout, 0.f);
                if ((int)op.hw[1].size() != op.cout)
                    throw FormatError("size of bias does not match");
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "RMSNormalization") {
                op.kind = OpKind::LayerNorm;
                op.rms = true;
                op.hw.resize(2);
                op.hw[0] = decode_floats(param(sc, c.layer, "scale"));
                op.cout = (int)op.hw[0].size();
                op.eps = (float)cfg.at("epsilon").number();
                const Value& ax = cfg.at("axis");
                if (ax.is_array())
                    for (const auto& a : ax.arr)
                        op.target_shape.push_back(a.integer());
                else
                    op.target_shape.push_back(ax.integer());
                result = add_op(std::move(op));
            } else if (cls == "GroupQueryAttention" || cls == "GroupedQueryAttention") {
                // import_model.hpp:1445-1466, layers/group_query_attention_layer.hpp.  Runs on the attention op of
                // MultiHeadAttention with the key / value kernels repeated once per query head of their group.
                op.kind = OpKind::MHA;
                const int hd = (int)cfg.at("head_dim").integer(), hq = (int)cfg.at("num_query_heads").integer(),
                          hkv = (int)cfg.at("num_key_value_heads").integer();
                op.use_bias = cfg.at("use_bias").boolean();
                const Value* ug = cfg.find("use_gate");
                op.gate = ug && ug->is_bool() && ug->boolean();
                if (hkv <= 0)
                    throw FormatError("num_key_value_heads must be > 0.");
                if (hq % hkv != 0)
                    throw FormatError("num_query_heads must be divisible by num_key_value_heads.");
                if (ins.size() != 2 && ins.size() != 3)
                    throw FormatError("GroupQueryAttention requires 2 or 3 inputs (query, value[, key]).");
                const Value& vals = param(sc, c.layer, "weights");
                const size_t step = op.use_bias ? 2 : 1, n_proj = op.gate ? 5 : 4;
                if (!vals.is_array() || vals.size() != step * n_proj)
                    throw FormatError("GroupQueryAttention: unexpected number of weights");
                std::vector<std::vector<float>> w;
                for (const auto& v : vals.arr)
                    w.push_back(decode_floats(v));
                op.heads = hq;
                op.dk = op.dv = hd;
                const int group = hq / hkv;
                int d_in = -1;
                // (D, heads, hd) -> [hq*hd][D], head h of the result read from head h / rep of the file
                auto kernel_t = [&](const std::vector<float>& k, int heads, int rep) {
                    if (k.size() % ((size_t)heads * hd) != 0)
                        throw FormatError("GroupQueryAttention: kernel size does not match the head layout");
                    const int d = (int)(k.size() / ((size_t)heads * hd));
                    if (d_in >= 0 && d != d_in)
                        throw FormatError("GroupQueryAttention kernels disagree on the input depth");
                    d_in = d;
                    std::vector<float> t((size_t)heads * rep * hd * d);
                    for (int h = 0; h < heads * rep; ++h)
                        for (int cc = 0; cc < hd; ++cc)
                            for (int i = 0; i < d; ++i)
                                t[((size_t)h * hd + cc) * d + i] = k[((size_t)i * heads + h / rep) * hd + cc];
                    return t;
                };
                auto bias_of = [&](size_t proj, int heads, int rep) {
                    std::vector<float> b((size_t)heads * rep * hd, 0.f);
                    if (op.use_bias) {
                        const std::vector<float>& src = w[proj * step + 1];
                        if (src.size() != (size_t)heads * hd)
                            throw FormatError("GroupQueryAttention: bias size does not match the head layout");
                        for (int h = 0; h < heads * rep; ++h)
                            for (int cc = 0; cc < hd; ++cc)
                                b[(size_t)h * hd + cc] = src[(size_t)(h / rep) * hd + cc];
                    }
                    return b;
                };
                const size_t vi = op.gate ? 3 : 2, oi = op.gate ? 4 : 3;
                op.hw.resize(op.gate ? 10 : 8);
                op.hw[0] = kernel_t(w[0], hq, 1);
                op.hw[1] = bias_of(0, hq, 1);
                op.hw[2] = kernel_t(w[step], hkv, group);
                op.hw[3] = bias_of(1, hkv, group);
                op.hw[4] = kernel_t(w[vi * step], hkv, group);
                op.hw[5] = bias_of(vi, hkv, group);
                op.d_in = d_in;
                const std::vector<float>& ow = w[oi * step]; // (hq, hd, Dout) -> [Dout][hq*hd]
                const int kin = hq * hd;
                if (ow.size() % (size_t)kin != 0)
                    throw FormatError("Invalid output kernel shape for GroupQueryAttention");
                op.dout = (int)(ow.size() / (size_t)kin);
                op.hw[6].resize(ow.size());
                for (int i = 0; i < kin; ++i)
                    for (int o2 = 0; o2 < op.dout; ++o2)
                        op.hw[6][(size_t)o2 * kin + i] = ow[(size_t)i * op.dout + o2];
                op.hw[7].assign((size_t)op.dout, 0.f);
                if (op.use_bias) {
                    if (w[oi * step + 1].size() != (size_t)op.dout)
                        throw FormatError("GroupQueryAttention: output bias size");
                    op.hw[7] = w[oi * step + 1];
                }
                if (op.gate) {
                    op.hw[8] = kernel_t(w[2 * step], hq, 1);
                    op.hw[9] = bias_of(2, hq, 1);
                }
                result = add_op(std::move(op));
            } else if (cls == "LayerNormalization") {
                op.kind = OpKind::LayerNorm;
                op.hw.resize(2);
                if (cfg.at("scale").boolean())
                    op.hw[0] = decode_floats(param(sc, c.layer, "gamma"));
                if (cfg.at("center").boolean())
                    op.hw[1] = decode_floats(param(sc, c.layer, "beta"));
                op.eps = (float)cfg.at("epsilon").number();
                if (!op.hw[0].empty() && !op.hw[1].empty() && op.hw[0].size() != op.hw[1].size())
                    throw FormatError("LayerNormalization: gamma and beta differ in size");
                op.cout = (int)std::max(op.hw[0].size(), op.hw[1].size());
                const Value& ax = cfg.at("axis");
                op.target_shape.clear();
                if (ax.is_array())
                    for (const auto& a : ax.arr)
                        op.target_shape.push_back(a.integer());
                else
                    op.target_shape.push_back(ax.integer());
                result = add_op(std::move(op));
            } else if (cls == "Activation") {
                result = activation_op(op.name, cfg.at("activation").str(), &cfg, ins[0]);
            } else if (kActivationLayers.count(cls)) {
                result = activation_op(op.name, kActivationLayers.at(cls), &cfg, ins[0]);
            } else if (cls == "PReLU") {
                op.kind = OpKind::PReLU;
                op.hw.resize(1);
                op.hw[0] = decode_floats(param(sc, c.layer, "alpha"));
                op.cout = (int)op.hw[0].size();
                if (const Value* sa = cfg.find("shared_axes"))
                    if (sa->is_array())
                        for (const auto& a : sa->arr)
                            op.shared_axes.push_back(a.integer());
                result = add_op(std::move(op));
            } else if (cls == "UpSampling2D" || cls == "UpSampling1D") {
                op.kind = OpKind::Resize;
                if (cls == "UpSampling1D") {
                    op.kh = 1;
                    op.kw = (int)cfg.at("size").integer();
                } else {
                    pair_from(cfg.at("size"), op.kh, op.kw);
                    const std::string ip = cfg.at("interpolation").str();
                    if (ip != "nearest" && ip != "bilinear")
                        throw FormatError("Invalid interpolation method: " + ip);
                    op.bilinear = ip == "bilinear";
                }
                if (op.kh < 1 || op.kw < 1)
                    throw FormatError("invalid upsampling factor");
                result = add_op(std::move(op));
            } else if (cls == "Cropping2D" || cls == "Cropping1D") {
                // import_model.hpp:1075-1115: ((top, bottom), (left, right)), or for 1-D (left, right)
                op.kind = OpKind::Crop;
                const Value& cr = cfg.at("cropping");
                if (!cr.is_array() || cr.size() != 2)
                    throw FormatError("invalid cropping format");
                if (cr.arr[0].is_array()) {
                    if (cr.arr[0].size() != 2 || cr.arr[1].size() != 2)
                        throw FormatError("invalid cropping format");
                    op.zp[0] = (int)cr.arr[0].at((size_t)0).integer();
                    op.zp[1] = (int)cr.arr[0].at(1).integer();
                    op.zp[2] = (int)cr.arr[1].at((size_t)0).integer();
                    op.zp[3] = (int)cr.arr[1].at(1).integer();
                } else {
                    op.zp[2] = (int)cr.at((size_t)0).integer();
                    op.zp[3] = (int)cr.at(1).integer();
                }
                result = add_op(std::move(op));
            } else if (cls == "Permute") {
                op.kind = OpKind::Permute;
                for (const auto& d : cfg.at("dims").arr)
                    op.target_shape.push_back(d.integer());
                result = add_op(std::move(op));
            } else if (cls == "ZeroPadding1D") {
                op.kind = OpKind::ZeroPad;
                const Value& p = cfg.at("padding");
                if (p.is_array() && p.size() == 2) {
                    op.zp[2] = (int)p.at((size_t)0).integer();
                    op.zp[3] = (int)p.at(1).integer();
                } else if (p.is_number()) {
                    op.zp[2] = op.zp[3] = (int)p.integer();
                } else
                    throw FormatError("invalid padding format");
                result = add_op(std::move(op));
            } else if (cls == "ZeroPadding2D") {
                op.kind = OpKind::ZeroPad;
                const Value& p = cfg.at("padding");
                if (!p.is_array() || p.size() != 2 || !p.arr[0].is_array() || p.arr[0].size() != 2 || p.arr[1].size() != 2)
                    throw FormatError("invalid padding format");
                op.zp[0] = (int)p.arr[0].at((size_t)0).integer();
                op.zp[1] = (int)p.arr[0].at(1).integer();
                op.zp[2] = (int)p.arr[1].at((size_t)0).integer();
                op.zp[3] = (int)p.arr[1].at(1).integer();
                result = add_op(std::move(op));
            } else if (cls == "MaxPooling2D" || cls == "AveragePooling2D" || cls == "MaxPooling1D" || cls == "AveragePooling1D") {
                op.kind = OpKind::Pool;
                op.pool_mode = cls[0] == 'M' ? 0 : 1;
                pair_from(cfg.at("pool_size"), op.kh, op.kw);
                const Value& st = cfg.at("strides");
                if (st.is_null()) {
                    op.sy = op.kh;
                    op.sx = op.kw;
                } else
                    pair_from(st, op.sy, op.sx);
                op.padding = padding_from(cfg.at("padding").str());
                result = add_op(std::move(op));
            } else if (cls == "GlobalAveragePooling2D" || cls == "GlobalMaxPooling2D" || cls == "GlobalAveragePooling1D"
                || cls == "GlobalMaxPooling1D") {
                op.kind = OpKind::GlobalPool;
                op.pool_mode = cls.find("Max") != std::string::npos ? 0 : 1;
                const Value* kd = cfg.find("keepdims");
                op.keepdims = kd && kd->is_bool() && kd->boolean();
                result = add_op(std::move(op));
            } else if (cls == "Add" || cls == "Multiply" || cls == "Subtract" || cls == "Average" || cls == "Maximum"
                || cls == "Minimum") {
                op.kind = OpKind::Add;
                op.combine = cls == "Multiply" ? FDX_COMBINE_MUL : cls == "Subtract" ? FDX_COMBINE_SUB
                    : cls == "Maximum"         ? FDX_COMBINE_MAX
                    : cls == "Minimum"         ? FDX_COMBINE_MIN
                                               : FDX_COMBINE_ADD;
                if (cls == "Subtract" && ins.size() != 2)
                    throw FormatError("subtract layer needs exactly two input tensors");
                if (cls == "Average")
                    op.scale = 1.0f / (float)ins.size(); // average_tensors: the sum times 1 / n (tensor.hpp:886-891)
                result = add_op(std::move(op));
            } else if (cls == "Concatenate") {
                op.kind = OpKind::Concat;
                op.axis = (int)cfg.at("axis").integer();
                result = add_op(std::move(op));
            } else if (cls == "EinsumDense") {
                // import_model.hpp:820-848
                op.kind = OpKind::Einsum;
                op.equation = cfg.at("equation").str();
                const Value* ba = cfg.find("bias_axes");
                op.bias_axes = ba && ba->is_string() ? ba->str() : "";
                op.full_out.push_back(-1); // batch slot
                if (const Value* os = cfg.find("output_shape")) {
                    if (os->is_array())
                        for (const auto& d : os->arr)
                            op.full_out.push_back(d.is_null() ? -1 : d.integer());
                    else if (!os->is_null())
                        op.full_out.push_back(os->integer());
                }
                for (const auto& d : param(sc, c.layer, "kernel_shape").arr)
                    op.kernel_dims.push_back(d.integer());
                op.hw.resize(2);
                op.hw[0] = decode_floats(param(sc, c.layer, "kernel"));
                if ((int64_t)op.hw[0].size() != volume(op.kernel_dims))
                    throw FormatError("EinsumDense: kernel values do not fill kernel_shape");
                EinsumSpec spec;
                std::string err;
                if (!spec.parse(op.equation, op.bias_axes, err))
                    throw FormatError(err);
                if (!op.bias_axes.empty())
                    op.hw[1] = decode_floats(param(sc, c.layer, "bias"));
                std::string n_chars;
                if (spec.gemm_form(&n_chars) && spec.ker.size() == op.kernel_dims.size()) {
                    // kernel [K][N] -> [N][K]; bias spread over the N characters
                    for (size_t i = 0; i < spec.ker.size(); ++i)
                        spec.size[spec.ker[i]] = op.kernel_dims[i];
                    const int64_t K = spec.volume_of(spec.summed), N = spec.volume_of(n_chars);
                    std::vector<float> t(op.hw[0].size());
                    for (int64_t k = 0; k < K; ++k)
                        for (int64_t n = 0; n < N; ++n)
                            t[(size_t)(n * K + k)] = op.hw[0][(size_t)(k * N + n)];
                    op.hw[0].swap(t);
                    std::vector<float> b((size_t)N, 0.f);
                    if (!spec.bias_chars.empty()) {
                        if ((int64_t)op.hw[1].size() != spec.volume_of(spec.bias_chars))
                            throw FormatError("EinsumDense: bias size does not match bias_axes");
                        for (int64_t n = 0; n < N; ++n) {
                            int64_t rem = n, off = 0;
                            for (size_t i = n_chars.size(); i-- > 0;) {
                                const int64_t ext = spec.size.at(n_chars[i]);
                                off += (rem % ext) * spec.stride_in(spec.bias_chars, n_chars[i]);
                                rem /= ext;
                            }
                            b[(size_t)n] = op.hw[1][(size_t)off];
                        }
                    }
                    op.hw[1].swap(b);
                    op.gemm = true;
                    op.n_in = (int)K;
                    op.units = (int)N;
                }
                result = with_fused_activation(add_op(std::move(op)), cfg);
            } else if (cls == "Embedding") {
                op.kind = OpKind::Embedding;
                op.input_dim = (int)cfg.at("input_dim").integer();
                op.output_dim = (int)cfg.at("output_dim").integer();
                op.hw.resize(1);
                op.hw[0] = decode_floats(param(sc, c.layer, "weights"));
                if (op.hw[0].size() != (size_t)op.input_dim * op.output_dim)
                    throw FormatError("embedding weight size does not match input_dim * output_dim");
                m.has_embedding = true;
                result = add_op(std::move(op));
            } else if (cls == "MultiHeadAttention") {
                op.kind = OpKind::MHA;
                op.heads = (int)cfg.at("num_heads").integer();
                op.dk = (int)cfg.at("key_dim").integer();
                op.dv = (int)cfg.at("value_dim").integer();
                op.use_bias = cfg.at("use_bias").boolean();
                if (ins.size() != 2 && ins.size() != 3)
                    throw FormatError("Invalid number of inputs for MultiHeadAttention layer.");
                const Value& shapes = param(sc, c.layer, "weight_shapes");
                const Value& vals = param(sc, c.layer, "weights");
                const size_t expect = op.use_bias ? 8 : 4;
                if (!shapes.is_array() || !vals.is_array() || shapes.size() != expect || vals.size() != expect)
                    throw FormatError("MultiHeadAttention expects q/k/v/output kernels (and biases)");
                std::vector<std::vector<float>> w;
                for (const auto& v : vals.arr)
                    w.push_back(decode_floats(v));
                const int step = op.use_bias ? 2 : 1;
                const int H = op.heads;
                // kernels arrive (D, H, dim): transpose to [H*dim][D], the B operand of the projection GEMM
                auto kernel_t = [&](const std::vector<float>& k, int dim, int& d_in) {
                    if (k.size() % ((size_t)H * dim) != 0)
                        throw FormatError("Invalid weights shape for attention head dimension.");
                    d_in = (int)(k.size() / ((size_t)H * dim));
                    std::vector<float> t(k.size());
                    const int n = H * dim;
                    for (int i = 0; i < d_in; ++i)
                        for (int o = 0; o < n; ++o)
                            t[(size_t)o * d_in + i] = k[(size_t)i * n + o];
                    return t;
                };
                auto bias_of = [&](int idx, int n) {
                    std::vector<float> b = op.use_bias ? w[(size_t)idx * step + 1] : std::vector<float>((size_t)n, 0.f);
                    if ((int)b.size() != n)
                        throw FormatError("Invalid biases shape for attention head dimension.");
                    return b;
                };
                op.hw.resize(8);
                int dq = 0, dkk = 0, dvv = 0;
                op.hw[0] = kernel_t(w[0], op.dk, dq);
                op.hw[1] = bias_of(0, H * op.dk);
                op.hw[2] = kernel_t(w[(size_t)step], op.dk, dkk);
                op.hw[3] = bias_of(1, H * op.dk);
                op.hw[4] = kernel_t(w[(size_t)2 * step], op.dv, dvv);
                op.hw[5] = bias_of(2, H * op.dv);
                if (dq != dkk || dq != dvv)
                    throw FormatError("MultiHeadAttention kernels disagree on the input depth");
                op.d_in = dq;
                const std::vector<float>& ow = w[(size_t)3 * step]; // (H, dv, Dout) = [H*dv][Dout] -> [Dout][H*dv]
                const int kin = H * op.dv;
                if (ow.size() % (size_t)kin != 0)
                    throw FormatError("Invalid output kernel shape for MultiHeadAttention");
                op.dout = (int)(ow.size() / (size_t)kin);
                op.hw[6].resize(ow.size());
                for (int i = 0; i < kin; ++i)
                    for (int o = 0; o < op.dout; ++o)
                        op.hw[6][(size_t)o * kin + i] = ow[(size_t)i * op.dout + o];
                op.hw[7] = bias_of(3, op.dout);
                result = add_op(std::move(op));
            } else if (cls == "Flatten") {
                op.kind = OpKind::View;
                op.flatten = true;
                result = add_op(std::move(op));
            } else if (cls == "Reshape") {
                op.kind = OpKind::View;
                for (const auto& d : cfg.at("target_shape").arr)
                    op.target_shape.push_back(d.integer());
                result = add_op(std::move(op));
            } else {
                throw Unsupported("unknown layer type: " + cls);
            }
            return sc.memo[key] = result;
        }
    };

    void replace_uses(fdx_model& m, int from, int to)
    {
        for (auto& o : m.ops) {
            for (auto& i : o.in)
                if (i == from)
                    i = to;
            if (o.residual == from)
                o.residual = to;
        }
        for (auto& o : m.outputs)
            if (o == from)
                o = to;
    }

    void count_consumers(fdx_model& m)
    {
        for (auto& o : m.ops)
            o.consumers = 0;
        for (auto& o : m.ops) {
            if (o.dead)
                continue;
            for (int i : o.in)
                m.ops[i].consumers++;
            if (o.residual >= 0)
                m.ops[o.residual].consumers++;
        }
        for (int o : m.outputs)
            m.ops[o].consumers++;
    }

    bool is_gemm_like(const Op& o) { return o.kind == OpKind::Conv2D || o.kind == OpKind::Dense; }
    bool fold_ln_requested(); // fdx_debug_force_ln_fold(1) is in force
    bool chain_requested();   // fdx_debug_force_chain(1) is in force

    fdx_status infer_shapes(const fdx_model& m, const std::vector<Shape>& in_shapes, std::vector<Shape>& shapes,
        const std::vector<int>& order);

} // namespace

std::vector<int> topo_order(const fdx_model& m)
{
    {
        std::vector<int> order;
        std::vector<char> seen(m.ops.size(), 0);
        std::function<void(int)> visit = [&](int i) {
            if (seen[i])
                return;
            seen[i] = 1;
            for (int p : m.ops[i].in)
                visit(p);
            if (m.ops[i].residual >= 0)
                visit(m.ops[i].residual);
            order.push_back(i);
        };
        for (int i : m.inputs)
            visit(i);
        for (int o : m.outputs)
            visit(o);
        return order;
    }
}

namespace {

    void fuse(fdx_model& m)
    {
        // shapes with every variable dimension set to a dummy extent decide which Adds are plain
        // (equal-shape) sums
        std::vector<Shape> dummy;
        for (const auto& s : m.in_decl) {
            Shape d = s;
            for (auto& v : d)
                if (v < 0)
                    v = 6;
            dummy.push_back(d);
        }
        std::vector<Shape> shapes;
        const bool have_shapes = infer_shapes(m, dummy, shapes, topo_order(m)) == FDX_OK;
        // Two tensors that agree under one dummy extent need not agree at run time (a variable dimension against a fixed
        // one of that extent, or two different variable dimensions): an Add only counts as an equal-shape sum if its
        // operands also agree with every variable dimension at a second extent and, where the graph accepts it, with
        // every variable dimension at an extent of its own.
        std::vector<Shape> shapes_b, shapes_c;
        bool have_b = false, have_c = false;
        {
            std::vector<Shape> dummy_b = m.in_decl, dummy_c = m.in_decl;
            int64_t next = 11;
            for (size_t i = 0; i < dummy_b.size(); ++i)
                for (size_t d = 0; d < dummy_b[i].size(); ++d)
                    if (dummy_b[i][d] < 0) {
                        dummy_b[i][d] = 7;
                        dummy_c[i][d] = next;
                        next += 2;
                    }
            have_b = infer_shapes(m, dummy_b, shapes_b, topo_order(m)) == FDX_OK;
            have_c = infer_shapes(m, dummy_c, shapes_c, topo_order(m)) == FDX_OK;
        }
        auto same_shape_always = [&](int x, int y) {
            return shapes[x] == shapes[y] && have_b && shapes_b[x] == shapes_b[y] && (!have_c || shapes_c[x] == shapes_c[y]);
        };

        count_consumers(m);
        // 1. BatchNormalization on the channel axis into the producing convolution / dense weights
        for (size_t i = 0; i < m.ops.size(); ++i) {
            Op& bn = m.ops[i];
            if (bn.dead || bn.kind != OpKind::Affine || bn.affine_scalar)
                continue;
            Op& p = m.ops[bn.in[0]];
            const bool producer_ok = (is_gemm_like(p) || p.kind == OpKind::DWConv2D) && p.act.kind == FDX_ACT_NONE
                && !p.softmax && p.consumers == 1 && p.residual < 0;
            if (!producer_ok || !have_shapes)
                continue;
            const int rank = (int)shapes[i].size();
            const int axis = bn.ln_axes < 0 ? bn.ln_axes + rank + 1 : bn.ln_axes;
            const int ch = p.kind == OpKind::Dense ? p.units : p.cout;
            if (axis != rank || bn.cout != ch)
                continue;
            const size_t per = p.hw[0].size() / (size_t)ch;
            if (p.kind == OpKind::DWConv2D) { // filter is [kh][kw][c]
                for (size_t t = 0; t < per; ++t)
                    for (int c = 0; c < ch; ++c)
                        p.hw[0][t * ch + c] *= bn.hw[0][c];
            } else { // [cout][k]
                for (int c = 0; c < ch; ++c)
                    for (size_t t = 0; t < per; ++t)
                        p.hw[0][(size_t)c * per + t] *= bn.hw[0][c];
            }
            for (int c = 0; c < ch; ++c)
                p.hw[1][c] = p.hw[1][c] * bn.hw[0][c] + bn.hw[1][c];
            bn.dead = true;
            replace_uses(m, (int)i, bn.in[0]);
            count_consumers(m);
        }
        // 2. stand-alone ReLU / GELU into the producer's epilogue
        for (size_t i = 0; i < m.ops.size(); ++i) {
            Op& a = m.ops[i];
            if (a.dead || a.kind != OpKind::Act || !(a.act.kind == FDX_ACT_RELU || a.act.kind == FDX_ACT_GELU))
                continue;
            Op& p = m.ops[a.in[0]];
            const bool ok = (is_gemm_like(p) || p.kind == OpKind::DWConv2D || p.kind == OpKind::Add || p.kind == OpKind::Affine
                                || p.kind == OpKind::Einsum)
                && p.act.kind == FDX_ACT_NONE && !p.softmax && p.consumers == 1;
            if (!ok)
                continue;
            p.act = a.act;
            a.dead = true;
            replace_uses(m, (int)i, a.in[0]);
            count_consumers(m);
        }
        // 3. ZeroPadding2D into the consumer's load predicate
        for (size_t i = 0; i < m.ops.size(); ++i) {
            Op& c = m.ops[i];
            if (c.dead || !(c.kind == OpKind::Conv2D || c.kind == OpKind::DWConv2D || c.kind == OpKind::Pool))
                continue;
            Op& z = m.ops[c.in[0]];
            if (z.dead || z.kind != OpKind::ZeroPad || z.consumers != 1)
                continue;
            for (int k = 0; k < 4; ++k)
                c.zp[k] += z.zp[k];
            c.in[0] = z.in[0];
            z.dead = true;
            count_consumers(m);
        }
        // 4. two-input equal-shape Add into the epilogue of the convolution / dense that feeds it
        for (size_t i = 0; i < m.ops.size() && have_shapes; ++i) {
            Op& add = m.ops[i];
            if (add.dead || add.kind != OpKind::Add || add.in.size() != 2 || add.in[0] == add.in[1] || add.combine != FDX_COMBINE_ADD
                || add.scale != 1.0f)
                continue;
            if (!same_shape_always(add.in[0], add.in[1]))
                continue;
            for (int side = 1; side >= 0; --side) {
                Op& p = m.ops[add.in[side]];
                // (an attention op ends in its output projection, a GEMM with the same epilogue)
                if ((is_gemm_like(p) || p.kind == OpKind::MHA) && p.consumers == 1 && p.residual < 0 && !p.softmax
                    && p.act.kind == FDX_ACT_NONE && !p.dead) {
                    p.residual = add.in[1 - side];
                    p.act = add.act;
                    add.dead = true;
                    replace_uses(m, (int)i, add.in[side]);
                    count_consumers(m);
                    break;
                }
            }
        }
        // 5. a residual operand that is itself a 1x1 convolution (the shortcut branch of a block that changes the channel
        // count or the resolution: Add(Conv2D(a), Conv2D(b))) joins the 1x1 stride-1 convolution that adds it.  The two
        // become one GEMM over both inputs' channels, and the shortcut's output is neither written nor read back.
        static const bool dual_on = [] { const char* e = std::getenv("FDX_DUAL_CONV"); return !(e && e[0] == '0'); }();
        for (size_t i = 0; i < m.ops.size() && have_shapes && dual_on; ++i) {
            Op& c = m.ops[i];
            auto plain_1x1 = [](const Op& o) {
                return !o.dead && o.kind == OpKind::Conv2D && o.kh == 1 && o.kw == 1 && o.dy == 1 && o.dx == 1 && o.zp[0] == 0 && o.zp[1] == 0
                    && o.zp[2] == 0 && o.zp[3] == 0 && !o.softmax && o.fuse_dw < 0 && o.fused_into < 0 && o.fuse_exp < 0 && o.exp_into < 0
                    && o.dual_cin == 0 && o.hw.size() == 2 && o.n_in > 0 && o.n_in % 16 == 0 && o.cout >= 64 && o.cout % 4 == 0
                    && o.hw[0].size() == (size_t)o.cout * (size_t)o.n_in && o.hw[1].size() == (size_t)o.cout;
            };
            if (c.residual < 0 || c.residual == c.in[0] || !plain_1x1(c) || c.sy != 1 || c.sx != 1)
                continue;
            Op& r = m.ops[c.residual];
            if (!plain_1x1(r) || r.cout != c.cout || r.act.kind != FDX_ACT_NONE || r.consumers != 1 || r.residual >= 0 || r.in.size() != 1)
                continue;
            const int k1 = c.n_in, k2 = r.n_in;
            c.hw.resize(6);
            c.hw[5].resize((size_t)c.cout * (size_t)(k1 + k2));
            for (int n = 0; n < c.cout; ++n) {
                std::copy_n(&c.hw[0][(size_t)n * k1], k1, &c.hw[5][(size_t)n * (k1 + k2)]);
                std::copy_n(&r.hw[0][(size_t)n * k2], k2, &c.hw[5][(size_t)n * (k1 + k2) + k1]);
                c.hw[1][n] += r.hw[1][n];
            }
            c.hw[0].clear(); // the joint filter serves both inputs
            c.dual_cin = k2;
            c.dual_sy = r.sy;
            c.dual_sx = r.sx;
            c.in.push_back(r.in[0]);
            c.residual = -1;
            r.dead = true;
            count_consumers(m);
        }
        // 7. a LayerNormalization over the last axis whose only readers are Dense layers and self-attention layers (all of
        // query, value and key): the readers are marked, and get their filters with gamma / beta folded in when the weights
        // are uploaded; a plan may then normalise inside their GEMMs and skip the LayerNormalization launch.  The op itself
        // and the readers' own filters stay (a decode session folds them its own way, and sizes the GEMM kernel does not
        // cover run as before).
        // (Only on request, FDX_LN_FOLD=1 or the test hook set when the model is loaded: on the benched encoder -- 8192 rows of
        // 512, 12 LayerNormalization launches of 11 us -- the statistics cost the two GEMMs that gather them 12 % of their
        // time, 0.7 % more per step than the launches they save; and the folded copies take as much memory as the filters.)
        static const bool ln_fold_env = [] { const char* e = std::getenv("FDX_LN_FOLD"); return e && e[0] == '1'; }();
        for (size_t i = 0; i < m.ops.size() && have_shapes && (ln_fold_env || fold_ln_requested()); ++i) {
            Op& ln = m.ops[i];
            if (ln.dead || ln.kind != OpKind::LayerNorm || ln.rms || ln.act.kind != FDX_ACT_NONE || ln.in.size() != 1 || ln.target_shape.size() != 1)
                continue;
            const Shape& xs = shapes[ln.in[0]];
            if (xs.empty())
                continue;
            const int64_t a = ln.target_shape[0];
            const int64_t C = xs.back();
            if (!(a == -1 || a == (int64_t)xs.size()) || C < 32 || C % 32 != 0)
                continue;
            if ((ln.hw.size() > 0 && !ln.hw[0].empty() && (int64_t)ln.hw[0].size() != C) || (ln.hw.size() > 1 && !ln.hw[1].empty() && (int64_t)ln.hw[1].size() != C))
                continue;
            bool is_output = false;
            for (int out : m.outputs)
                is_output = is_output || out == (int)i;
            std::vector<int> readers;
            bool ok = !is_output;
            for (size_t q = 0; q < m.ops.size() && ok; ++q) {
                const Op& r = m.ops[q];
                if (r.dead)
                    continue;
                const bool reads = std::find(r.in.begin(), r.in.end(), (int)i) != r.in.end();
                if (r.residual == (int)i)
                    ok = false;
                if (!reads)
                    continue;
                if (r.kind == OpKind::Dense && r.in.size() == 1 && r.n_in == C && r.hw.size() == 2 && r.ln_src < 0
                    && r.hw[0].size() == (size_t)r.units * (size_t)C && r.hw[1].size() == (size_t)r.units && r.units % 4 == 0 && r.units >= 16) {
                    readers.push_back((int)q);
                } else if (r.kind == OpKind::MHA && r.ln_src < 0 && !r.gate && r.d_in == C && r.hw.size() >= 6 && r.in.size() >= 2
                    && r.in[0] == (int)i && r.in[1] == (int)i && (r.in.size() == 2 || r.in[2] == (int)i) && (r.heads * r.dk) % 4 == 0
                    && (r.heads * r.dv) % 4 == 0) {
                    readers.push_back((int)q);
                } else {
                    ok = false;
                }
            }
            if (!ok || readers.empty())
                continue;
            for (int q : readers) {
                m.ops[q].ln_src = (int)i;
                m.ops[q].ln_eps = ln.eps;
            }
        }
        // 6. a 1x1 stride-1 convolution whose result another 1x1 stride-1 convolution reads (a block's last convolution, with
        // its Add and ReLU in the epilogue, and the next block's first): marked as a pair that one launch can run, the
        // second convolution taking the first's result from LDS (conv1x1_chain_launch).  Whether a plan does so is decided
        // when the plan is made.
        static const bool chain_env = [] { const char* e = std::getenv("FDX_CHAIN"); return e && e[0] == '1'; }();
        // (pairs are marked, and their packed filters kept, only on request: FDX_CHAIN=1, or the test hook set when the model
        // is loaded)
        for (size_t i = 0; i < m.ops.size() && have_shapes && (chain_env || chain_requested()); ++i) {
            Op& d = m.ops[i];
            auto gemm_1x1 = [](const Op& o) {
                return !o.dead && o.kind == OpKind::Conv2D && o.kh == 1 && o.kw == 1 && o.sy == 1 && o.sx == 1 && o.dy == 1 && o.dx == 1
                    && o.zp[0] == 0 && o.zp[1] == 0 && o.zp[2] == 0 && o.zp[3] == 0 && !o.softmax && o.fuse_dw < 0 && o.fused_into < 0
                    && o.fuse_exp < 0 && o.exp_into < 0 && o.chain < 0 && o.chained_from < 0 && o.n_in > 0
                    && (o.act.kind == FDX_ACT_NONE || o.act.kind == FDX_ACT_RELU || o.act.kind == FDX_ACT_GELU)
                    && o.hw.size() >= 2 && o.hw[1].size() == (size_t)o.cout;
            };
            if (!gemm_1x1(d) || d.in.size() != 1 || d.residual >= 0 || d.dual_cin > 0 || d.hw.size() != 2
                || d.hw[0].size() != (size_t)d.cout * (size_t)d.n_in)
                continue;
            Op& c = m.ops[d.in[0]];
            if (!gemm_1x1(c) || c.cout != d.n_in || !chain_supported(c.n_in, c.dual_cin, c.cout, d.cout))
                continue;
            const bool dual = c.dual_cin > 0;
            if (dual ? !(c.hw.size() == 6 && c.hw[5].size() == (size_t)c.cout * (size_t)(c.n_in + c.dual_cin))
                     : !(c.hw.size() == 2 && c.hw[0].size() == (size_t)c.cout * (size_t)c.n_in))
                continue;
            if (shapes[d.in[0]].size() != 3)
                continue;
            const int k = c.n_in + c.dual_cin;
            c.hw.resize(7);
            c.hw[6].resize(chain_first_floats(c.cout, k));
            chain_pack_first(dual ? c.hw[5].data() : c.hw[0].data(), c.cout, k, c.hw[6].data());
            d.hw.resize(7);
            d.hw[6].resize(chain_second_floats(c.cout, d.cout));
            chain_pack_second(d.hw[0].data(), c.cout, d.cout, d.hw[6].data());
            c.chain = (int)i;
            d.chained_from = d.in[0];
        }
        // last: depthwise 3x3 convolutions whose only consumer is a 1x1 convolution (the second half of an
        // inverted-residual block, a SeparableConv2D) are marked; whether the pair runs as one launch is decided per plan
        // by timing both forms
        static const bool dwpw_on = [] { const char* e = std::getenv("FDX_DWPW"); return !(e && e[0] == '0'); }();
        for (size_t i = 0; dwpw_on && i < m.ops.size(); ++i) {
            Op& c = m.ops[i];
            if (c.dead || c.kind != OpKind::Conv2D || c.kh != 1 || c.kw != 1 || c.sy != 1 || c.sx != 1 || c.softmax
                || c.zp[0] || c.zp[1] || c.zp[2] || c.zp[3] || c.in.empty() || c.dual_cin > 0 || c.chain >= 0 || c.chained_from >= 0)
                continue;
            Op& d = m.ops[c.in[0]];
            if (d.dead || d.kind != OpKind::DWConv2D || d.kh != 3 || d.kw != 3 || d.dy != 1 || d.dx != 1 || d.sy != d.sx
                || d.consumers != 1 || d.softmax || d.residual >= 0 || d.fused_into >= 0 || c.residual == c.in[0])
                continue;
            if (!fdx_dwconv_pointwise_supported(d.cout, c.cout, d.sy))
                continue;
            c.fuse_dw = c.in[0];
            d.fused_into = (int)i;
            // ... and the 1x1 expansion in front of the depthwise convolution, where one launch covers the whole block
            if (d.in.empty())
                continue;
            Op& e = m.ops[d.in[0]];
            const bool act_ok = e.act.kind == FDX_ACT_NONE || e.act.kind == FDX_ACT_RELU || e.act.kind == FDX_ACT_GELU;
            if (e.dead || e.kind != OpKind::Conv2D || e.softmax || e.residual >= 0 || e.consumers != 1 || e.fuse_dw >= 0 || e.exp_into >= 0
                || e.dual_cin > 0 || e.chain >= 0 || e.chained_from >= 0 || !act_ok || e.hw.empty() || e.cout <= 0 || e.hw[0].size() % (size_t)e.cout != 0)
                continue;
            const bool pointwise = e.kh == 1 && e.kw == 1 && e.sy == 1 && e.sx == 1 && !e.zp[0] && !e.zp[1] && !e.zp[2] && !e.zp[3];
            // ... or the small convolution on the image a MobileNet-like network starts with (3x3 / 2 on RGB)
            const bool stem = !pointwise && e.kh == e.kw && e.sy == e.sx && e.dy == 1 && e.dx == 1 && e.n_in > 0
                && fdx_stem_block_supported(e.n_in, e.kh, e.cout, c.cout, d.sy);
            if ((pointwise && fdx_inverted_residual_supported((int)(e.hw[0].size() / (size_t)e.cout), e.cout, c.cout, d.sy)) || stem) {
                c.fuse_exp = d.in[0];
                e.exp_into = (int)i;
            }
        }
    }

    fdx_status upload(fdx_model& m)
    {
        // gamma / beta of the LayerNormalization ops some reader folds into its filter (the op's own arrays are released when
        // it is uploaded, before its readers' turn)
        std::map<int, std::pair<std::vector<float>, std::vector<float>>> ln_affine;
        for (auto& o : m.ops)
            if (!o.dead && o.ln_src >= 0 && !ln_affine.count(o.ln_src)) {
                const Op& ln = m.ops[(size_t)o.ln_src];
                ln_affine[o.ln_src] = { ln.hw.size() > 0 ? ln.hw[0] : std::vector<float>(), ln.hw.size() > 1 ? ln.hw[1] : std::vector<float>() };
            }
        // filter [n][k] with gamma folded in, bias with beta folded in, row sums of the folded filter
        auto fold_ln = [&](int ln_idx, const std::vector<float>& w, const std::vector<float>& b, int n, int k, std::vector<float>& wf,
                           std::vector<float>& bf, std::vector<float>& ws) {
            const auto& gb = ln_affine[ln_idx];
            wf.resize((size_t)n * k);
            bf.assign((size_t)n, 0.f);
            ws.assign((size_t)n, 0.f);
            for (int r = 0; r < n; ++r) {
                double sum = 0.0, shift = b.empty() ? 0.0 : (double)b[(size_t)r];
                for (int c = 0; c < k; ++c) {
                    const float wv = w[(size_t)r * k + c];
                    const float f = gb.first.empty() ? wv : wv * gb.first[(size_t)c];
                    wf[(size_t)r * k + c] = f;
                    sum += (double)f;
                    if (!gb.second.empty())
                        shift += (double)wv * (double)gb.second[(size_t)c];
                }
                ws[(size_t)r] = (float)sum;
                bf[(size_t)r] = (float)shift;
            }
        };
        for (auto& o : m.ops) {
            if (o.dead) {
                o.hw.clear();
                continue;
            }
            // stem convolutions get a third weight array: the filter in its space-to-depth layout
            static const bool s2d_on = [] { const char* e = std::getenv("FDX_S2D"); return !(e && e[0] == '0'); }();
            if (s2d_on && o.kind == OpKind::Conv2D && o.hw.size() == 2
                && fdx_conv2d_s2d_eligible(o.n_in, o.kh, o.kw, o.sy, o.sx, o.dy, o.dx, o.cout)) {
                o.hw.emplace_back(fdx_conv2d_s2d_weight_floats(o.cout, o.n_in, o.kh));
                if (fdx_conv2d_s2d_prepare(o.hw[0].data(), o.cout, o.n_in, o.kh, o.hw[2].data()) != FDX_OK)
                    return FDX_ERR_INVALID;
            }
            // pointwise convolutions whose channel count is a multiple of 4 but not of 16 (24, 40, 72 ...): a fourth weight
            // array holds the filter rows padded with zero taps to the next multiple of 16, see conv1x1_padded_launch
            if (o.kind == OpKind::Conv2D && o.hw.size() == 2 && o.kh == 1 && o.kw == 1 && o.sy == 1 && o.sx == 1 && o.n_in % 4 == 0
                && o.n_in % 16 != 0 && o.cout % 4 == 0 && o.cout >= 64) {
                const int kp = (o.n_in + 15) / 16 * 16;
                o.hw.resize(4);
                o.hw[3].assign((size_t)o.cout * kp, 0.f);
                for (int n = 0; n < o.cout; ++n)
                    std::copy_n(&o.hw[0][(size_t)n * o.n_in], o.n_in, &o.hw[3][(size_t)n * kp]);
            }
            // 3x3 stride-1 convolutions get a fifth weight array: the filter in the Winograd F(2x2, 3x3) domain; whether a
            // plan runs the direct or the Winograd kernel is decided per shape by timing both
            static const bool wino_on = [] { const char* e = std::getenv("FDX_WINOGRAD"); return !(e && e[0] == '0'); }();
            if (wino_on && o.kind == OpKind::Conv2D && o.hw.size() == 2 && o.kh == 3 && o.kw == 3 && o.sy == 1 && o.sx == 1 && o.dy == 1
                && o.dx == 1 && !o.softmax && fdx_conv2d_winograd_supported(o.n_in, o.cout)) {
                o.hw.resize(5);
                o.hw[4].resize(fdx_conv2d_winograd_weight_floats(o.cout, o.n_in));
                if (fdx_conv2d_winograd_prepare(o.hw[0].data(), o.cout, o.n_in, o.hw[4].data()) != FDX_OK)
                    return FDX_ERR_INVALID;
            }
            // self-attention (query, value and key are one tensor): the three projections become one GEMM over the
            // stacked kernels, whose column blocks the attention core then reads in place
            if (o.kind == OpKind::MHA && o.hw.size() >= 6 && o.in.size() >= 2 && o.in[0] == o.in[1]
                && (o.in.size() == 2 || o.in[2] == o.in[0]) && (o.heads * o.dk) % 4 == 0 && (o.heads * o.dv) % 4 == 0) {
                o.hw.resize(std::max<size_t>(o.hw.size(), 12));
                for (int part = 0; part < 3; ++part) {
                    o.hw[10].insert(o.hw[10].end(), o.hw[(size_t)2 * part].begin(), o.hw[(size_t)2 * part].end());
                    o.hw[11].insert(o.hw[11].end(), o.hw[(size_t)2 * part + 1].begin(), o.hw[(size_t)2 * part + 1].end());
                }
            }
            if (o.ln_src >= 0 && o.kind == OpKind::Dense && o.hw.size() == 2) {
                o.hw.resize(5);
                fold_ln(o.ln_src, o.hw[0], o.hw[1], o.units, o.n_in, o.hw[2], o.hw[3], o.hw[4]);
            } else if (o.ln_src >= 0 && o.kind == OpKind::MHA && o.hw.size() >= 12 && !o.hw[10].empty()) {
                const int nt = 2 * o.heads * o.dk + o.heads * o.dv;
                o.hw.resize(15);
                fold_ln(o.ln_src, o.hw[10], o.hw[11], nt, o.d_in, o.hw[12], o.hw[13], o.hw[14]);
            } else {
                o.ln_src = -1; // (an attention op whose projections were not stacked, ...: it reads the LayerNormalization's result)
            }
            o.dw.assign(o.hw.size(), nullptr);
            for (size_t i = 0; i < o.hw.size(); ++i) {
                if (o.hw[i].empty())
                    continue;
                float* d = nullptr;
                FDX_HIP(hipMalloc(&d, o.hw[i].size() * sizeof(float)));
                m.device_allocs.push_back(d);
                FDX_HIP(hipMemcpy(d, o.hw[i].data(), o.hw[i].size() * sizeof(float), hipMemcpyHostToDevice));
                o.dw[i] = d;
            }
            o.hw.clear();
            o.hw.shrink_to_fit();
        }
        FDX_HIP(hipMalloc(&m.err_flag, sizeof(int)));
        FDX_HIP(zero_device(m.err_flag, sizeof(int)));
        return FDX_OK;
    }

    // (height, width, depth) view of a rank-3 sample, or of a rank-2 (width, depth) one with height 1; empty otherwise
    Shape hwc(const Shape& s)
    {
        if (s.size() == 3)
            return s;
        if (s.size() == 2)
            return { 1, s[0], s[1] };
        return {};
    }

    fdx_status window(int h, int w, const Op& o, bool dilated, int* g)
    {
        const int ekh = dilated ? (o.kh - 1) * o.dy + 1 : o.kh, ekw = dilated ? (o.kw - 1) * o.dx + 1 : o.kw;
        return fdx_window_geometry(h + o.zp[0] + o.zp[1], w + o.zp[2] + o.zp[3], ekh, ekw, o.sy, o.sx, o.padding, g);
    }

    fdx_status infer_shapes(const fdx_model& m, const std::vector<Shape>& in_shapes, std::vector<Shape>& shapes,
        const std::vector<int>& order)
    {
        shapes.assign(m.ops.size(), Shape());
        for (int idx : order) {
            const Op& o = m.ops[idx];
            if (o.dead)
                continue;
            Shape& out = shapes[idx];
            const Shape* in0 = o.in.empty() ? nullptr : &shapes[o.in[0]];
            int g[6];
            switch (o.kind) {
            case OpKind::Input:
                out = in_shapes[o.input_index];
                break;
            case OpKind::Conv2D:
            case OpKind::DWConv2D: {
                Shape s = *in0;
                if (s.size() == 2)
                    s.insert(s.begin(), 1); // 1-D convolution: height 1
                FDX_REQUIRE(s.size() == 3, "%s: convolution needs a (height, width, depth) input", o.name.c_str());
                FDX_REQUIRE(s[2] == o.n_in, "invalid filter depth");
                if (window((int)s[0], (int)s[1], o, true, g) != FDX_OK)
                    return FDX_ERR_INVALID;
                FDX_REQUIRE(g[4] > 0 && g[5] > 0, "%s: empty convolution output", o.name.c_str());
                out = { g[4], g[5], o.cout };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Dense:
                FDX_REQUIRE(!in0->empty() && in0->back() == o.n_in, "%s: Dense input depth %lld does not match weights (%d)",
                    o.name.c_str(), in0->empty() ? 0LL : (long long)in0->back(), o.n_in);
                out = *in0;
                out.back() = o.units;
                break;
            case OpKind::Affine:
            case OpKind::Act:
            case OpKind::Softmax:
            case OpKind::LayerNorm:
            case OpKind::PReLU:
                out = *in0;
                break;
            case OpKind::ZeroPad: {
                const Shape s3 = hwc(*in0);
                FDX_REQUIRE(!s3.empty(), "%s: zero padding needs a rank-2 or rank-3 input", o.name.c_str());
                out = { s3[0] + o.zp[0] + o.zp[1], s3[1] + o.zp[2] + o.zp[3], s3[2] };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Pool: {
                const Shape s3 = hwc(*in0);
                FDX_REQUIRE(!s3.empty(), "%s: pooling needs a rank-2 or rank-3 input", o.name.c_str());
                if (window((int)s3[0], (int)s3[1], o, false, g) != FDX_OK)
                    return FDX_ERR_INVALID;
                FDX_REQUIRE(g[4] > 0 && g[5] > 0, "%s: empty pooling output", o.name.c_str());
                out = { g[4], g[5], s3[2] };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Resize: {
                const Shape s3 = hwc(*in0);
                FDX_REQUIRE(!s3.empty(), "%s: upsampling needs a rank-2 or rank-3 input", o.name.c_str());
                out = { s3[0] * o.kh, s3[1] * o.kw, s3[2] };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Dilate: {
                const Shape s3 = hwc(*in0);
                FDX_REQUIRE(!s3.empty(), "Invalid rank for dilation");
                out = { (s3[0] - 1) * o.kh + 1 + (o.trailing ? o.kh - 1 : 0), (s3[1] - 1) * o.kw + 1 + (o.trailing ? o.kw - 1 : 0), s3[2] };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Crop: {
                const Shape s3 = hwc(*in0);
                FDX_REQUIRE(!s3.empty(), "%s: cropping needs a rank-2 or rank-3 input", o.name.c_str());
                FDX_REQUIRE(o.zp[0] + o.zp[1] < s3[0] && o.zp[2] + o.zp[3] < s3[1], "%s: cropping removes the whole tensor", o.name.c_str());
                out = { s3[0] - o.zp[0] - o.zp[1], s3[1] - o.zp[2] - o.zp[3], s3[2] };
                if (in0->size() == 2)
                    out.erase(out.begin());
                break;
            }
            case OpKind::Permute: {
                FDX_REQUIRE(o.target_shape.size() == in0->size(), "%s: Permute dims do not match the input rank", o.name.c_str());
                out.clear();
                std::vector<char> seen(in0->size(), 0);
                for (int64_t d : o.target_shape) {
                    FDX_REQUIRE(d >= 1 && d <= (int64_t)in0->size() && !seen[(size_t)d - 1], "Invalid dims for permute.");
                    seen[(size_t)d - 1] = 1;
                    out.push_back((*in0)[(size_t)d - 1]);
                }
                break;
            }
            case OpKind::GlobalPool:
                FDX_REQUIRE(in0->size() >= 2, "%s: global pooling needs rank >= 2", o.name.c_str());
                if (o.keepdims) {
                    out.assign(in0->size(), 1);
                    out.back() = in0->back();
                } else
                    out = { in0->back() };
                break;
            case OpKind::Add: {
                // tensor.hpp:642-660: right-aligned axes must be equal or 1; the result has the larger rank
                out = *in0;
                for (size_t k = 1; k < o.in.size(); ++k) {
                    const Shape& b = shapes[o.in[k]];
                    if (b == out)
                        continue;
                    Shape r(std::max(out.size(), b.size()), 1);
                    for (size_t d = 0; d < r.size(); ++d) {
                        const int64_t x = d < out.size() ? out[out.size() - 1 - d] : 1, y = d < b.size() ? b[b.size() - 1 - d] : 1;
                        FDX_REQUIRE(x == y || x == 1 || y == 1, "Invalid shapes for combining tensors.");
                        r[r.size() - 1 - d] = std::max(x, y);
                    }
                    out = r;
                }
                break;
            }
            case OpKind::Concat: {
                // tensor.hpp:459-483: the axis counts from the first input's rank
                const int rank = (int)in0->size();
                int axis = o.axis < 0 ? o.axis + rank + 1 : o.axis;
                FDX_REQUIRE(axis >= 1 && axis <= rank, "Invalid axis (%d) for tensor concatenation.", o.axis);
                out = *in0;
                for (size_t k = 1; k < o.in.size(); ++k) {
                    const Shape& b = shapes[o.in[k]];
                    FDX_REQUIRE(b.size() == out.size(), "%s: Concatenate inputs differ in rank", o.name.c_str());
                    for (int d = 0; d < rank; ++d)
                        FDX_REQUIRE(d == axis - 1 || b[(size_t)d] == out[(size_t)d], "%s: Concatenate inputs differ off the axis",
                            o.name.c_str());
                    out[(size_t)axis - 1] += b[(size_t)axis - 1];
                }
                break;
            }
            case OpKind::Host: {
                const fdx_host_layer& hl = m.host_layers[(size_t)o.host_index];
                std::vector<int> ranks;
                std::vector<int64_t> dims5;
                std::vector<const float*> ptrs(o.in.size(), nullptr);
                std::vector<std::vector<float>> zeros;
                for (int i : o.in) {
                    const Shape& s = shapes[i];
                    FDX_REQUIRE(!s.empty() && s.size() <= 5, "%s: custom layer inputs must have rank 1..5", o.name.c_str());
                    ranks.push_back((int)s.size());
                    for (size_t k = 0; k < 5; ++k)
                        dims5.push_back(k < 5 - s.size() ? 1 : s[k - (5 - s.size())]);
                    zeros.emplace_back((size_t)volume(s), 0.f);
                }
                for (size_t i = 0; i < ptrs.size(); ++i)
                    ptrs[i] = zeros[i].data();
                int orank = 0;
                int64_t od[5] = { 1, 1, 1, 1, 1 };
                if (hl.vt.apply(hl.instance, (int)o.in.size(), ptrs.data(), ranks.data(), dims5.data(), nullptr, &orank, od) != FDX_OK) {
                    set_error("%s: custom layer failed on the shape pass: %s", o.name.c_str(), fdx_last_error());
                    return FDX_ERR_INVALID;
                }
                FDX_REQUIRE(orank >= 1 && orank <= 5, "%s: custom layer returned rank %d", o.name.c_str(), orank);
                out.assign(od + 5 - orank, od + 5);
                for (auto d : out)
                    FDX_REQUIRE(d > 0, "%s: custom layer returned an empty shape", o.name.c_str());
                break;
            }
            case OpKind::Einsum: {
                EinsumSpec spec;
                std::string err;
                Shape dims = *in0;
                if (!spec.parse(o.equation, o.bias_axes, err) || !(dims.size() < spec.lhs.size())) {
                    set_error("%s: %s", o.name.c_str(), err.empty() ? "EinsumDense: input rank exceeds lhs char count." : err.c_str());
                    return FDX_ERR_INVALID;
                }
                if (!spec.derive_sizes(o.kernel_dims, dims, o.full_out, err)) {
                    set_error("%s: %s", o.name.c_str(), err.c_str());
                    return FDX_ERR_INVALID;
                }
                out.clear();
                for (size_t i = 1; i < spec.rhs.size(); ++i)
                    out.push_back(spec.size.at(spec.rhs[i]));
                FDX_REQUIRE(out.size() <= 5, "%s: EinsumDense output rank above 5", o.name.c_str());
                break;
            }
            case OpKind::Embedding:
                FDX_REQUIRE(in0->size() == 1, "size_dim_5, size_dim_4, height and width dimension must be 1");
                out = { (*in0)[0], o.output_dim };
                break;
            case OpKind::MHA: {
                const Shape& q = shapes[o.in[0]];
                const Shape& v = shapes[o.in[1]];
                const Shape& k = shapes[o.in.size() > 2 ? o.in[2] : o.in[1]];
                FDX_REQUIRE(q.size() == 2 && v.size() == 2 && k.size() == 2 && q[1] == v[1] && q[1] == k[1] && v[0] == k[0],
                    "Invalid shapes; need a query tensor of shape (B, T, dim) and a value/key tensor of shape (B, S, dim).");
                FDX_REQUIRE(q[1] == o.d_in, "%s: attention input depth does not match the kernels", o.name.c_str());
                out = { q[0], o.dout };
                break;
            }
            case OpKind::View:
                if (o.flatten)
                    out = { volume(*in0) };
                else if (!o.target_shape.empty()) {
                    out = o.target_shape;
                    int64_t known = 1, unknown = -1;
                    for (size_t d = 0; d < out.size(); ++d)
                        if (out[d] < 0)
                            unknown = (int64_t)d;
                        else
                            known *= out[d];
                    if (unknown >= 0)
                        out[(size_t)unknown] = volume(*in0) / std::max<int64_t>(known, 1);
                    FDX_REQUIRE(volume(out) == volume(*in0), "Invalid target shape");
                } else
                    out = *in0;
                break;
            }
        }
        return FDX_OK;
    }

    double op_flops(const Op& o, const Shape& out, const std::vector<Shape>& shapes, int batch)
    {
        switch (o.kind) {
        case OpKind::Conv2D: return 2.0 * batch * volume(out) * (o.kh * o.kw * o.n_in + o.dual_cin);
        case OpKind::Dense: return 2.0 * batch * volume(out) * o.n_in;
        case OpKind::Einsum: return o.gemm ? 2.0 * batch * volume(out) * o.n_in : 0.0;
        case OpKind::MHA: {
            const double t = (double)shapes[o.in[0]][0], s = (double)shapes[o.in[1]][0];
            return 2.0 * batch * (t * o.d_in * o.heads * o.dk + s * o.d_in * o.heads * (o.dk + o.dv)
                       + (double)o.heads * t * s * (o.dk + o.dv) + t * o.heads * o.dv * o.dout);
        }
        default: return 0.0;
        }
    }

} // namespace

// test hook: -1 = a plan times both forms of a depthwise + 1x1 pair, 0 = always two launches, 1 = always one
static int g_force_dw_fusion = -1;

extern "C" fdx_status fdx_debug_force_dw_fusion(int mode)
{
    FDX_REQUIRE(mode >= -1 && mode <= 2, "fdx_debug_force_dw_fusion: mode must be -1, 0, 1 or 2");
    g_force_dw_fusion = mode;
    return FDX_OK;
}

// test hook: 0 = plans built from now on run every LayerNormalization as a launch of its own, 1 = they normalise inside the
// readers' GEMMs where those are Dense / self-attention layers of a size the kernel covers, -1 = as the environment says
// (FDX_LN_FOLD=1: inside the GEMMs; otherwise launches of their own)
static int g_force_ln_fold = -1;

namespace {
bool fold_ln_requested() { return g_force_ln_fold == 1; }
}

extern "C" fdx_status fdx_debug_force_ln_fold(int mode)
{
    FDX_REQUIRE(mode >= -1 && mode <= 1, "fdx_debug_force_ln_fold: mode must be -1, 0 or 1");
    g_force_ln_fold = mode;
    return FDX_OK;
}

// test hook: -1 = plans run a pair of 1x1 convolutions as one launch where the closed rule says so, 0 = never, 1 = wherever
// the kernel covers the pair
static int g_force_chain = -1;

namespace {
bool chain_requested() { return g_force_chain == 1; }
}

extern "C" fdx_status fdx_debug_force_chain(int mode)
{
    FDX_REQUIRE(mode >= -1 && mode <= 1, "fdx_debug_force_chain: mode must be -1, 0 or 1");
    g_force_chain = mode;
    return FDX_OK;
}

// test hook: -1 = a plan times the direct and the Winograd kernel of a 3x3 stride-1 convolution, 0 = always direct, 1 = Winograd
// wherever it applies
static int g_force_winograd = -1;

extern "C" fdx_status fdx_debug_force_winograd(int mode)
{
    FDX_REQUIRE(mode >= -1 && mode <= 1, "fdx_debug_force_winograd: mode must be -1, 0 or 1");
    g_force_winograd = mode;
    return FDX_OK;
}

fdx_status get_plan(fdx_model* m, int batch, const std::vector<Shape>& in_shapes, Plan** out)
{
    for (size_t i = 0; i < m->plans.size(); ++i)
        if (m->plans[i]->batch == batch && m->plans[i]->in_shapes == in_shapes) {
            if (i != 0)
                std::rotate(m->plans.begin(), m->plans.begin() + (std::ptrdiff_t)i, m->plans.begin() + (std::ptrdiff_t)i + 1);
            *out = m->plans[0].get();
            return FDX_OK;
        }
    if (m->plans.size() >= fdx_model::kMaxPlans) {
        // the least recently used plan gives its buffers back before the new one asks for its own
        FDX_HIP(hipStreamSynchronize(stream()));
        m->plans.pop_back();
    }
    std::unique_ptr<Plan> p(new Plan);
    p->batch = batch;
    p->in_shapes = in_shapes;
    p->order = topo_order(*m);
    fdx_status st = infer_shapes(*m, in_shapes, p->shapes, p->order);
    if (st != FDX_OK)
        return st;
    const size_t n = m->ops.size();
    p->out.assign(n, nullptr);
    p->block_of.assign(n, -1);
    p->last_use.assign(n, -1);
    p->temps.assign(n, {});
    p->dw_fused.assign(n, g_force_dw_fusion < 0 ? 0 : (g_force_dw_fusion == 1 ? 1 : (g_force_dw_fusion == 2 ? 3 : 2)));
    p->conv_form.assign(n, (signed char)g_force_winograd);
    // Pairs of 1x1 convolutions that one launch can run: off unless asked for (FDX_CHAIN=1 or the test hook).  Measured on
    // ResNet50's 56 x 56 stage at batch 64, the one launch takes as long as the two it replaces where the first convolution
    // adds a residual (178 us either way) and longer where it sums two inputs (218 against 175 us): what it saves in
    // memory traffic it loses to its serial phases at two workgroups per CU.
    p->chain_on.assign(n, 0);
    p->chain_done.assign(n, 0);
    for (int idx : p->order) {
        const Op& o = m->ops[idx];
        if (o.dead || o.chain < 0 || m->ops[o.chain].dead || p->shapes[idx].size() != 3)
            continue;
        const int64_t rows = (int64_t)batch * p->shapes[idx][0] * p->shapes[idx][1];
        static const bool chain_default = [] { const char* e = std::getenv("FDX_CHAIN"); return e && e[0] == '1'; }();
        const bool wanted = g_force_chain >= 0 ? g_force_chain != 0 : (chain_default && rows >= 65536);
        p->chain_on[idx] = wanted ? 1 : 0;
    }
    // LayerNormalization ops whose readers all normalise inside their own GEMM in this plan: no launch of their own
    p->ln_fold_on.assign(n, 0);
    p->ln_skip.assign(n, 0);
    for (int idx : p->order) {
        const Op& ln = m->ops[idx];
        static const bool ln_fold_default = [] { const char* e = std::getenv("FDX_LN_FOLD"); return e && e[0] == '1'; }();
        if (ln.dead || ln.kind != OpKind::LayerNorm || !(g_force_ln_fold == 1 || (g_force_ln_fold < 0 && ln_fold_default)))
            continue;
        bool all = true, any = false;
        for (int q : p->order) {
            const Op& r = m->ops[q];
            if (r.dead || std::find(r.in.begin(), r.in.end(), idx) == r.in.end())
                continue;
            any = true;
            const Shape& xs = p->shapes[ln.in[0]];
            const int64_t rows = xs.empty() ? 0 : (int64_t)batch * volume(xs) / xs.back();
            const int n_out = r.kind == OpKind::Dense ? r.units : 2 * r.heads * r.dk + r.heads * r.dv;
            const size_t folded = r.kind == OpKind::Dense ? 2 : 12;
            all = all && r.ln_src == idx && r.dw.size() > folded + 2 && r.dw[folded] && !xs.empty() && rows > 16
                && gemm_ln_supported(rows, n_out, (int)xs.back());
        }
        if (!any || !all)
            continue;
        p->ln_skip[idx] = 1;
        for (int q : p->order)
            if (!m->ops[q].dead && m->ops[q].ln_src == idx)
                p->ln_fold_on[q] = 1;
    }
    std::vector<int> s2d_ops;
    // lifetime: position of the last consumer; a View extends the life of the buffer it aliases
    std::vector<int> root(n);
    for (int idx : p->order) {
        const Op& o = m->ops[idx];
        root[idx] = (o.kind == OpKind::View) ? root[o.in[0]] : idx;
    }
    for (size_t pos = 0; pos < p->order.size(); ++pos) {
        const Op& o = m->ops[p->order[pos]];
        for (int i : o.in)
            p->last_use[root[i]] = (int)pos;
        if (o.residual >= 0)
            p->last_use[root[o.residual]] = (int)pos;
        if (o.ln_src >= 0 && p->ln_fold_on[p->order[pos]]) // normalising inside its GEMM, the op reads the LayerNormalization's input
            for (int i : m->ops[o.ln_src].in)
                p->last_use[root[i]] = (int)pos;
        if (o.fuse_dw >= 0) // run as one launch, the pair reads the depthwise convolution's input here
            for (int i : m->ops[o.fuse_dw].in)
                p->last_use[root[i]] = (int)pos;
        if (o.fuse_exp >= 0) // ... and the whole block the expansion's input
            for (int i : m->ops[o.fuse_exp].in)
                p->last_use[root[i]] = (int)pos;
    }
    for (int o : m->outputs)
        p->last_use[root[o]] = 1 << 30;
    for (int i : m->inputs)
        p->last_use[root[i]] = 1 << 30; // input staging buffers persist across calls
    // Plans whose one large input may arrive from host memory in pieces run their first ops piece by piece behind the copy
    // (predict_impl); that needs the results of those ops in blocks of their own, so the blocks of the ops that hold the
    // first fifth of the model's arithmetic are not recycled among them: they are released together behind that prefix.
    size_t hold_until = 0;
    if (m->inputs.size() == 1 && batch >= 8 && sizeof(float) * (size_t)batch * (size_t)volume(in_shapes[0]) >= ((size_t)4 << 20)) {
        double total = 0;
        for (int idx : p->order)
            total += op_flops(m->ops[idx], p->shapes[idx], p->shapes, batch);
        double sum = 0;
        for (size_t pos = 0; pos < p->order.size() && sum < total / 5; ++pos) {
            sum += op_flops(m->ops[p->order[pos]], p->shapes[p->order[pos]], p->shapes, batch);
            hold_until = pos + 1;
        }
        if (hold_until == p->order.size())
            hold_until = 0; // a model this shallow gains nothing
    }
    for (size_t pos = 0; pos < p->order.size(); ++pos) {
        const int idx = p->order[pos];
        const Op& o = m->ops[idx];
        if (o.kind == OpKind::View) {
            p->out[idx] = p->out[o.in[0]];
        } else {
            const size_t bytes = sizeof(float) * (size_t)batch * (size_t)volume(p->shapes[idx]);
            if (!p->out[idx]) // (the second convolution of a pair run as one launch got its block with the first)
                p->out[idx] = plan_alloc(*p, bytes, &p->block_of[idx]);
            if (!p->out[idx]) {
                set_error("out of device memory while planning %s", o.name.c_str());
                return FDX_ERR_HIP;
            }
            if (o.chain >= 0 && p->chain_on[idx]) { // this op's launch also writes its consumer's result
                const int d = o.chain;
                p->out[d] = plan_alloc(*p, sizeof(float) * (size_t)batch * (size_t)volume(p->shapes[d]), &p->block_of[d]);
                if (!p->out[d]) {
                    set_error("out of device memory while planning %s", m->ops[d].name.c_str());
                    return FDX_ERR_HIP;
                }
            }
        }
        if (o.kind == OpKind::Conv2D && o.dw.size() > 2 && o.dw[2] && p->shapes[idx].size() == 3)
            s2d_ops.push_back(idx); // scratch placed after the activations, see below
        if (o.kind == OpKind::MHA) { // per-op scratch: placed while inputs and output are live, free again afterwards
            const int64_t T = p->shapes[o.in[0]][0], S = p->shapes[o.in[1]][0];
            const size_t nk = (size_t)o.heads * o.dk, nv = (size_t)o.heads * o.dv, fb = sizeof(float) * (size_t)batch;
            const bool stacked = o.dw.size() > 11 && o.dw[10]; // one buffer holds [q | k | v] per row
            const size_t sizes[6] = { stacked ? fb * T * (2 * nk + nv) : fb * T * nk, stacked ? (size_t)256 : fb * S * nk,
                stacked ? (size_t)256 : fb * S * nv, fb * T * nv,
                fdx_mha_scratch_bytes(batch, o.heads, (int)T, (int)S, o.dv), o.gate ? fb * T * nv : (size_t)256 };
            std::vector<int> held;
            for (size_t sz : sizes) {
                int b = -1;
                float* t = plan_alloc(*p, sz, &b);
                if (!t) {
                    set_error("out of device memory while planning %s", o.name.c_str());
                    return FDX_ERR_HIP;
                }
                p->temps[idx].push_back(t);
                held.push_back(b);
            }
            for (int b : held)
                p->blocks[b].busy = false;
        }
        p->flops += op_flops(o, p->shapes[idx], p->shapes, batch);
        // release buffers whose last consumer is this op (the op's own output is already placed, so a
        // producer never writes over one of its live inputs)
        if (pos + 1 >= hold_until) {
            // (at the end of the held prefix: everything whose last reader lies inside it)
            for (size_t q = 0; q < n; ++q)
                if (p->block_of[q] >= 0 && p->blocks[p->block_of[q]].busy
                    && (p->last_use[q] == (int)pos || (pos + 1 == hold_until && p->last_use[q] < (int)pos)))
                    p->blocks[p->block_of[q]].busy = false;
            if (p->last_use[idx] < 0 && p->block_of[idx] >= 0) // produced but never read
                p->blocks[p->block_of[idx]].busy = false;
        }
    }
    // The space-to-depth scratch of stem convolutions gets blocks of its own, allocated last, so that it does not
    // change which blocks the activations land in.
    for (int idx : s2d_ops) {
        const Op& o = m->ops[idx];
        Block b;
        b.bytes = fdx_conv2d_s2d_scratch_bytes(batch, (int)p->shapes[idx][0], (int)p->shapes[idx][1], o.n_in, o.kh);
        if (hipMalloc(&b.p, b.bytes) != hipSuccess) {
            set_error("out of device memory while planning %s", o.name.c_str());
            return FDX_ERR_HIP;
        }
        b.busy = true;
        p->blocks.push_back(b);
        p->temps[idx].push_back(static_cast<float*>(b.p));
    }
    // With nothing to be timed, the direct-against-Winograd choice of every 3x3 stride-1 convolution is made here, from the
    // table or the closed rule, so that the first execution of the plan already runs what every later one runs.
    if (tune_frozen())
        for (int idx : p->order) {
            const Op& o = m->ops[idx];
            if (o.dead || o.kind != OpKind::Conv2D || !(o.dw.size() > 4 && o.dw[4]) || p->conv_form[idx] >= 0)
                continue;
            const Shape& is = p->shapes[o.in[0]];
            if (is.size() != 3)
                continue;
            int g[6];
            if (window((int)is[0], (int)is[1], o, true, g) != FDX_OK)
                continue;
            TuneKey key;
            std::memset(&key, 0, sizeof key);
            key.conv = 3; key.M = batch * g[4] * g[5]; key.N = o.cout; key.K = 9 * (int)is[2]; key.Cin = (int)is[2];
            key.kh = (int)is[0]; key.kw = (int)is[1]; key.sy = g[0] + o.zp[0]; key.sx = g[2] + o.zp[2]; key.batch = batch;
            key.res = o.residual >= 0;
            int known = 0;
            const bool listed = tune_lookup(key, &known);
            p->conv_form[idx] = (listed ? known == 1 : 2.0 * key.M * (double)key.N * key.K >= 1e9) ? 1 : 0;
        }
    m->plans.insert(m->plans.begin(), std::move(p));
    *out = m->plans[0].get();
    return FDX_OK;
}

namespace {

    fdx_act to_c(const Act& a) { return { a.kind, a.max_value, a.negative_slope, a.threshold }; }

    // First execution of a 3x3 stride-1 convolution that has a Winograd filter: the direct and the Winograd kernel are
    // timed on the real operands (both leave the same result, up to rounding, in the output buffer), the plan remembers
    // the faster one and the tuner's table keeps it per shape, so that an exported table pins it too.
    fdx_status choose_conv_form(fdx_model& m, Plan& p, int idx, const float* in0, int h, int w, int c, const int* g, const float* res,
        const fdx_act* actp, float* out)
    {
        const Op& o = m.ops[idx];
        const int B = p.batch;
        auto run = [&](int form) -> fdx_status {
            if (form == 1)
                return fdx_conv2d_winograd_nhwc_f32(in0, B, h, w, c, o.dw[4], o.dw[1], o.cout, g[0] + o.zp[0], g[2] + o.zp[2], g[4], g[5], res,
                    actp, out);
            return fdx_conv2d_nhwc_f32(in0, B, h, w, c, o.dw[0], o.dw[1], o.cout, o.kh, o.kw, o.sy, o.sx, o.dy, o.dx, g[0] + o.zp[0],
                g[2] + o.zp[2], g[4], g[5], res, actp, out);
        };
        TuneKey key;
        std::memset(&key, 0, sizeof key);
        key.conv = 3;
        key.M = B * g[4] * g[5];
        key.N = o.cout;
        key.K = 9 * c;
        key.Cin = c;
        key.kh = h;
        key.kw = w;
        key.sy = g[0] + o.zp[0];
        key.sx = g[2] + o.zp[2];
        key.batch = B;
        key.res = res != nullptr;
        int known = 0;
        hipEvent_t e0 = nullptr, e1 = nullptr;
        const bool listed = tune_lookup(key, &known);
        if (listed || tune_frozen() || hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) {
            if (e0)
                (void)hipEventDestroy(e0);
            // Nothing is timed and the shape is not in the table: the Winograd kernel from a gigaflop of direct-sum work
            // up (every 3x3 layer of ResNet50 from batch 5; timed, it wins all four of its shapes at batch 64 by 1.4-1.8
            // times), the direct kernel below that, where a launch is too short for the kernel's fixed costs to pay.
            const bool by_rule = 2.0 * key.M * (double)key.N * key.K >= 1e9;
            p.conv_form[idx] = (listed ? known == 1 : by_rule) ? 1 : 0;
            fdx_status st = run(p.conv_form[idx]);
            if (st == FDX_ERR_UNSUPPORTED && p.conv_form[idx] == 1) {
                p.conv_form[idx] = 0;
                st = run(0);
            }
            return st;
        }
        float ms[2] = { 1e30f, 1e30f };
        fdx_status st = FDX_OK;
        for (int form = 0; form < 2 && st == FDX_OK; ++form) {
            st = run(form); // warm-up (the direct kernel picks its tile here); tells whether the launcher takes the shape
            if (st == FDX_ERR_UNSUPPORTED && form == 1) {
                st = FDX_OK;
                continue;
            }
            if (st == FDX_OK && form == 0)
                tune_settle_clock([&] { return run(0) == FDX_OK; });
            for (int round = 0; round < 3 && st == FDX_OK; ++round) {
                (void)hipEventRecord(e0, stream());
                for (int r = 0; r < 3 && st == FDX_OK; ++r)
                    st = run(form);
                (void)hipEventRecord(e1, stream());
                float t = 1e30f;
                if (hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&t, e0, e1) == hipSuccess && t < ms[form])
                    ms[form] = t;
            }
        }
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        tune_mark();
        if (st != FDX_OK)
            return st;
        const int best = ms[1] < ms[0] ? 1 : 0;
        static const bool log_picks = [] { const char* e = std::getenv("FDX_TUNE_LOG"); return e && e[0] == '1'; }();
        if (log_picks)
            std::fprintf(stderr, "[fdx tune] %s: direct %.1f us, Winograd %.1f us\n", o.name.c_str(), ms[0] * 1e3f / 3, ms[1] * 1e3f / 3);
        p.conv_form[idx] = (signed char)best;
        tune_store(key, best);
        return run(best);
    }

    fdx_status run_op(fdx_model& m, Plan& p, int idx)
    {
        const Op& o = m.ops[idx];
        const int B = p.batch;
        const Shape& os = p.shapes[idx];
        float* out = p.out[idx];
        const float* in0 = o.in.empty() ? nullptr : p.out[o.in[0]];
        const Shape* is = o.in.empty() ? nullptr : &p.shapes[o.in[0]];
        const fdx_act act = to_c(o.act);
        const fdx_act* actp = o.act.kind == FDX_ACT_NONE ? nullptr : &act;
        const float* res = o.residual >= 0 ? p.out[o.residual] : nullptr;
        int g[6];
        fdx_status st = FDX_OK;
        switch (o.kind) {
        case OpKind::Input:
        case OpKind::View:
            return FDX_OK;
        case OpKind::Conv2D:
        case OpKind::DWConv2D: {
            const bool one_d = is->size() == 2;
            const int h = one_d ? 1 : (int)(*is)[0], w = (int)(*is)[one_d ? 0 : 1], c = (int)is->back();
            if ((st = window(h, w, o, true, g)) != FDX_OK)
                return st;
            if (o.kind == OpKind::Conv2D && o.chained_from >= 0 && p.chain_done[idx]) {
                p.chain_done[idx] = 0; // produced by the launch of the convolution in front
                break;
            }
            if (o.kind == OpKind::Conv2D && o.chain >= 0 && p.chain_on[idx] && o.dw.size() > 6 && o.dw[6]) {
                const Op& d = m.ops[o.chain];
                const fdx_act act2 = to_c(d.act);
                const bool dual = o.dual_cin > 0;
                const Shape* s2 = dual ? &p.shapes[o.in[1]] : nullptr;
                if ((!dual || (s2->size() == 3 && (*s2)[2] == o.dual_cin && ((*s2)[0] + o.dual_sy - 1) / o.dual_sy == g[4]
                                  && ((*s2)[1] + o.dual_sx - 1) / o.dual_sx == g[5]))
                    && !one_d && d.dw.size() > 6 && d.dw[6] && p.out[o.chain]) {
                    st = conv1x1_chain_launch(in0, B, g[4], g[5], c, dual ? p.out[o.in[1]] : nullptr, dual ? (int)(*s2)[0] : 0,
                        dual ? (int)(*s2)[1] : 0, dual ? o.dual_cin : 0, o.dual_sy, o.dual_sx, o.dual_cin, o.dw[6], o.dw[1], res, actp, o.cout,
                        out, d.dw[6], d.dw[1], d.act.kind == FDX_ACT_NONE ? nullptr : &act2, d.cout, p.out[o.chain]);
                    if (st == FDX_OK)
                        p.chain_done[o.chain] = 1;
                    if (st != FDX_ERR_UNSUPPORTED)
                        break;
                }
            }
            if (o.kind == OpKind::Conv2D && o.dual_cin > 0) {
                const Shape& s2 = p.shapes[o.in[1]];
                FDX_REQUIRE(o.dw.size() > 5 && o.dw[5] && s2.size() == 3 && s2[2] == o.dual_cin && !one_d, "%s: bad two-input convolution",
                    o.name.c_str());
                // (what the absorbed convolution would have produced must be what the other one produces: the Add of the
                // two needs equal shapes, layers/add_layer.hpp:20-29)
                FDX_REQUIRE((s2[0] + o.dual_sy - 1) / o.dual_sy == g[4] && (s2[1] + o.dual_sx - 1) / o.dual_sx == g[5],
                    "%s: the two convolutions of the sum give different shapes", o.name.c_str());
                st = conv1x1_dual_launch(in0, B, g[4], g[5], c, p.out[o.in[1]], (int)s2[0], (int)s2[1], o.dual_cin, o.dual_sy, o.dual_sx,
                    o.dw[5], o.dw[1], o.cout, actp, out);
                break;
            }
            if (o.kind == OpKind::Conv2D && o.dw.size() > 3 && o.dw[3] && g[0] + o.zp[0] == 0 && g[2] + o.zp[2] == 0 && g[4] == h && g[5] == w) {
                st = conv1x1_padded_launch(in0, (int64_t)B * h * w, c, o.dw[3], (c + 15) / 16 * 16, o.dw[1], o.cout, res, actp, out);
                if (st != FDX_ERR_UNSUPPORTED)
                    break;
            }
            if (o.kind == OpKind::Conv2D && o.dw.size() > 4 && o.dw[4]) {
                if (p.conv_form[idx] < 0) {
                    st = choose_conv_form(m, p, idx, in0, h, w, c, g, res, actp, out);
                    break; // the chosen form ran last and left its result
                }
                if (p.conv_form[idx] == 1) {
                    st = fdx_conv2d_winograd_nhwc_f32(in0, B, h, w, c, o.dw[4], o.dw[1], o.cout, g[0] + o.zp[0], g[2] + o.zp[2], g[4], g[5], res,
                        actp, out);
                    if (st != FDX_ERR_UNSUPPORTED)
                        break;
                }
            }
            if (o.kind == OpKind::Conv2D && !p.temps[idx].empty())
                st = fdx_conv2d_s2d_nhwc_f32(in0, B, h, w, c, o.dw[2], o.dw[1], o.cout, o.kh, g[0] + o.zp[0], g[2] + o.zp[2], g[4], g[5],
                    res, actp, p.temps[idx][0], out);
            else if (o.kind == OpKind::Conv2D)
                st = fdx_conv2d_nhwc_f32(in0, B, h, w, c, o.dw[0], o.dw[1], o.cout, o.kh, o.kw, o.sy, o.sx, o.dy, o.dx,
                    g[0] + o.zp[0], g[2] + o.zp[2], g[4], g[5], res, actp, out);
            else
                st = fdx_dwconv2d_nhwc_f32(in0, B, h, w, c, o.dw[0], o.dw[1], o.kh, o.kw, o.sy, o.sx, o.dy, o.dx,
                    g[0] + o.zp[0], g[2] + o.zp[2], g[4], g[5], actp, out);
            break;
        }
        case OpKind::Dense: {
            const int64_t rows = (int64_t)B * volume(*is) / o.n_in;
            FDX_REQUIRE(rows < (1LL << 31), "%s: too many rows", o.name.c_str());
            if (o.ln_src >= 0 && p.ln_fold_on[idx]) { // the LayerNormalization in front happens inside the GEMM
                st = gemm_ln_launch(p.out[m.ops[o.ln_src].in[0]], rows, o.n_in, o.dw[2], o.dw[3], o.dw[4], o.ln_eps, res, actp, out, o.units);
                break;
            }
            st = fdx_gemm_bias_act_f32(in0, o.n_in, o.dw[0], o.n_in, (int)rows, o.units, o.n_in, 1.0f, o.dw[1], 0, res, actp,
                out, o.units, nullptr);
            break;
        }
        case OpKind::Affine: {
            if (o.affine_scalar) { // one (scale, shift) pair for every element
                st = fdx_channel_affine_f32(in0, (size_t)B * (size_t)volume(*is), 1, o.dw[0], o.dw[1], actp, out);
                break;
            }
            const int rank = (int)is->size();
            const int axis = o.ln_axes < 0 ? o.ln_axes + rank + 1 : o.ln_axes;
            if (axis != rank || is->back() != o.cout) {
                set_error("%s: %s is supported on the last axis only", o.name.c_str(), o.cls.c_str());
                return FDX_ERR_UNSUPPORTED;
            }
            st = fdx_channel_affine_f32(in0, (size_t)B * (size_t)volume(*is) / (size_t)o.cout, o.cout, o.dw[0], o.dw[1], actp, out);
            break;
        }
        case OpKind::LayerNorm: {
            if (p.ln_skip[idx])
                return FDX_OK; // every reader normalises inside its own GEMM
            // axes are 1-based positions in the sample's own rank (negative from the end)
            const int rank = (int)is->size();
            int64_t dims5[5] = { 1, 1, 1, 1, 1 };
            for (int k = 0; k < rank; ++k)
                dims5[5 - rank + k] = (*is)[(size_t)k];
            unsigned mask = 0;
            int64_t count = 1;
            for (int64_t a : o.target_shape) {
                a = a < 0 ? a + rank + 1 : a;
                FDX_REQUIRE(a >= 1 && a <= rank, "%s: LayerNormalization axis out of range", o.name.c_str());
                const int pos = 5 - rank + (int)a - 1;
                if (!((mask >> pos) & 1u))
                    count *= dims5[pos];
                mask |= 1u << pos;
            }
            FDX_REQUIRE(o.cout == 0 || o.cout == count, "%s: gamma / beta do not match the normalised axes",
                o.name.c_str());
            st = o.rms ? fdx_rmsnorm_axes_f32(in0, B, dims5, mask, o.dw[0], o.eps, out)
                       : fdx_layernorm_axes_f32(in0, B, dims5, mask, o.dw[0], o.dw[1], o.eps, out);
            break;
        }
        case OpKind::Act:
            st = fdx_activation_f32(in0, (size_t)B * (size_t)volume(*is), actp, out);
            break;
        case OpKind::Softmax:
            st = fdx_softmax_f32(in0, (int64_t)B * volume(*is) / is->back(), (int)is->back(), 0, 0, out);
            if (st == FDX_OK && o.log_after) { // log_softmax = log(softmax(x)) (layers/log_softmax_layer.hpp)
                const fdx_act lg = { FDX_ACT_LOG, 0.f, 0.f, 0.f };
                st = fdx_activation_f32(out, (size_t)B * (size_t)volume(*is), &lg, out);
            }
            break;
        case OpKind::PReLU: {
            // layers/prelu_layer.hpp:29-70: alpha is laid out over (height, width, depth) with the shared axes collapsed;
            // shared axis numbers shift up when the sample has no height (and no width) axis of its own
            FDX_REQUIRE(is->size() <= 3, "%s: PReLU needs rank <= 3", o.name.c_str());
            int64_t xd[5] = { 1, 1, 1, 1, 1 };
            for (size_t d = 0; d < is->size(); ++d)
                xd[5 - is->size() + d] = (*is)[d];
            bool shared[4] = { false, false, false, false };
            int64_t shift = 0;
            for (int64_t a : o.shared_axes) {
                if ((a == 1 && xd[2] == 1) || (a == 2 && xd[3] == 1))
                    ++shift;
                const int64_t ax = a + shift;
                if (ax >= 1 && ax <= 3)
                    shared[ax] = true;
            }
            int64_t ad[5] = { 1, 1, shared[1] ? 1 : xd[2], shared[2] ? 1 : xd[3], shared[3] ? 1 : xd[4] };
            FDX_REQUIRE(ad[2] * ad[3] * ad[4] <= o.cout, "%s: PReLU alpha holds %d values, the input needs %lld", o.name.c_str(), o.cout,
                (long long)(ad[2] * ad[3] * ad[4]));
            st = fdx_broadcast_combine_f32(FDX_COMBINE_PRELU, in0, xd, o.dw[0], ad, 1, B, 1.0f, actp, out, nullptr);
            break;
        }
        case OpKind::ZeroPad: {
            const Shape s3 = hwc(*is);
            st = fdx_zero_pad2d_nhwc_f32(in0, B, (int)s3[0], (int)s3[1], (int)s3[2], o.zp[0], o.zp[1], o.zp[2], o.zp[3], out);
            break;
        }
        case OpKind::Pool: {
            const Shape s3 = hwc(*is);
            if ((st = window((int)s3[0], (int)s3[1], o, false, g)) != FDX_OK)
                return st;
            st = fdx_pool2d_nhwc_f32(in0, B, (int)s3[0], (int)s3[1], (int)s3[2], o.kh, o.kw, o.sy, o.sx, g[0] + o.zp[0],
                g[2] + o.zp[2], o.zp[0], o.zp[2], o.zp[1], o.zp[3], g[4], g[5], o.pool_mode, out);
            break;
        }
        case OpKind::Resize: {
            const Shape s3 = hwc(*is);
            st = fdx_upsample2d_nhwc_f32(in0, B, (int)s3[0], (int)s3[1], (int)s3[2], o.kh, o.kw, o.bilinear ? 1 : 0, out);
            break;
        }
        case OpKind::Dilate: {
            const Shape s3 = hwc(*is);
            st = fdx_dilate2d_nhwc_f32(in0, B, (int)s3[0], (int)s3[1], (int)s3[2], o.kh, o.kw, o.trailing ? 1 : 0, out);
            break;
        }
        case OpKind::Crop: {
            const Shape s3 = hwc(*is);
            st = fdx_crop2d_nhwc_f32(in0, B, (int)s3[0], (int)s3[1], (int)s3[2], o.zp[0], o.zp[1], o.zp[2], o.zp[3], out);
            break;
        }
        case OpKind::Permute: {
            int perm[5];
            for (size_t d = 0; d < o.target_shape.size(); ++d)
                perm[d] = (int)o.target_shape[d] - 1;
            st = fdx_permute_f32(in0, B, (int)is->size(), is->data(), perm, out);
            break;
        }
        case OpKind::GlobalPool:
            st = fdx_global_pool_f32(in0, B, (int)(volume(*is) / is->back()), (int)is->back(), o.pool_mode, out);
            break;
        case OpKind::Add: {
            // left fold of the layer's operation (tensor.hpp:677-690); the last step carries the scale of Average and
            // the fused activation
            const float* acc = in0;
            Shape acc_shape = *is;
            if (o.combine == FDX_COMBINE_MAX || o.combine == FDX_COMBINE_MIN)
                for (int i : o.in)
                    FDX_REQUIRE(p.shapes[i] == *is, "all tensors must have the same size");
            for (size_t k = 1; k < o.in.size() && st == FDX_OK; ++k) {
                const float* b = p.out[o.in[k]];
                const Shape& bs = p.shapes[o.in[k]];
                const bool last = k + 1 == o.in.size();
                const fdx_act* a = last ? actp : nullptr;
                const float scale = last ? o.scale : 1.0f;
                if (bs == acc_shape && o.combine == FDX_COMBINE_ADD && scale == 1.0f) {
                    const size_t n = (size_t)B * (size_t)volume(bs);
                    st = fdx_eltwise_add_f32(acc, b, n, n, a, out);
                } else {
                    int64_t ad[5] = { 1, 1, 1, 1, 1 }, bd[5] = { 1, 1, 1, 1, 1 }, od[5];
                    for (size_t d = 0; d < acc_shape.size(); ++d)
                        ad[5 - acc_shape.size() + d] = acc_shape[d];
                    for (size_t d = 0; d < bs.size(); ++d)
                        bd[5 - bs.size() + d] = bs[d];
                    // the running result may already live in `out`; it is only read in place when it has the output's shape
                    if (acc == out) {
                        bool same = true;
                        for (int d = 0; d < 5; ++d)
                            same = same && ad[d] >= bd[d];
                        FDX_REQUIRE(same, "%s: this chain of broadcasts needs a temporary", o.name.c_str());
                    }
                    st = fdx_broadcast_combine_f32(o.combine, acc, ad, b, bd, 0, B, scale, a, out, od);
                    Shape r(std::max(acc_shape.size(), bs.size()));
                    for (size_t d = 0; d < r.size(); ++d)
                        r[d] = od[5 - r.size() + d];
                    acc_shape = r;
                }
                acc = out;
            }
            if (o.in.size() == 1)
                st = fdx_activation_f32(in0, (size_t)B * (size_t)volume(*is), actp, out);
            break;
        }
        case OpKind::Concat: {
            const int rank = (int)is->size();
            const int axis = (o.axis < 0 ? o.axis + rank + 1 : o.axis) - 1;
            int64_t outer = B;
            for (int d = 0; d < axis; ++d)
                outer *= (*is)[(size_t)d];
            std::vector<const float*> ptrs;
            std::vector<int64_t> inner;
            for (int i : o.in) {
                const Shape& s = p.shapes[i];
                int64_t v = 1;
                for (int d = axis; d < rank; ++d)
                    v *= s[(size_t)d];
                ptrs.push_back(p.out[i]);
                inner.push_back(v);
            }
            st = fdx_concat_f32(ptrs.data(), (int)ptrs.size(), inner.data(), outer, out);
            if (st == FDX_OK && actp)
                st = fdx_activation_f32(out, (size_t)B * (size_t)volume(os), actp, out);
            break;
        }
        case OpKind::Host: {
            // drain the stream, run the layer on the host sample by sample, hand the result back to the device
            const fdx_host_layer& hl = m.host_layers[(size_t)o.host_index];
            const size_t n_in = o.in.size();
            std::vector<std::vector<float>> hin(n_in);
            std::vector<int> ranks;
            std::vector<int64_t> dims5;
            std::vector<int64_t> vols;
            for (size_t i = 0; i < n_in; ++i) {
                const Shape& s = p.shapes[o.in[i]];
                vols.push_back(volume(s));
                hin[i].resize((size_t)B * (size_t)vols[i]);
                FDX_HIP(hipMemcpyAsync(hin[i].data(), p.out[o.in[i]], hin[i].size() * sizeof(float), hipMemcpyDeviceToHost, stream()));
                ranks.push_back((int)s.size());
                for (size_t k = 0; k < 5; ++k)
                    dims5.push_back(k < 5 - s.size() ? 1 : s[k - (5 - s.size())]);
            }
            FDX_HIP(hipStreamSynchronize(stream()));
            const int64_t ovol = volume(os);
            std::vector<float> hout((size_t)B * (size_t)ovol);
            std::vector<const float*> ptrs(n_in);
            for (int b = 0; b < B; ++b) {
                for (size_t i = 0; i < n_in; ++i)
                    ptrs[i] = hin[i].data() + (size_t)b * (size_t)vols[i];
                int orank = 0;
                int64_t od[5] = { 1, 1, 1, 1, 1 };
                if (hl.vt.apply(hl.instance, (int)n_in, ptrs.data(), ranks.data(), dims5.data(), hout.data() + (size_t)b * (size_t)ovol,
                        &orank, od) != FDX_OK) {
                    set_error("%s: custom layer failed: %s", o.name.c_str(), fdx_last_error());
                    return FDX_ERR_INVALID;
                }
                FDX_REQUIRE(orank == (int)os.size() && Shape(od + 5 - orank, od + 5) == os,
                    "%s: custom layer changed its output shape between calls", o.name.c_str());
            }
            FDX_HIP(hipMemcpyAsync(out, hout.data(), hout.size() * sizeof(float), hipMemcpyHostToDevice, stream()));
            FDX_HIP(hipStreamSynchronize(stream()));
            if (actp)
                st = fdx_activation_f32(out, (size_t)B * (size_t)ovol, actp, out);
            break;
        }
        case OpKind::Einsum: {
            if (o.gemm) {
                const int64_t rows = (int64_t)B * volume(*is) / o.n_in;
                FDX_REQUIRE(rows < (1LL << 31), "%s: too many rows", o.name.c_str());
                st = fdx_gemm_bias_act_f32(in0, o.n_in, o.dw[0], o.n_in, (int)rows, o.units, o.n_in, 1.0f, o.dw[1], 0, res, actp, out,
                    o.units, nullptr);
            } else {
                // the leading lhs character is the batch: `B` samples back to back
                EinsumSpec spec;
                std::string err;
                spec.parse(o.equation, o.bias_axes, err);
                Shape dims = *is;
                while (dims.size() + 1 < spec.lhs.size())
                    dims.insert(dims.begin(), 1);
                dims.insert(dims.begin(), B);
                Shape full = o.full_out;
                if (!spec.derive_sizes(o.kernel_dims, dims, full, err)) {
                    set_error("%s: %s", o.name.c_str(), err.c_str());
                    return FDX_ERR_INVALID;
                }
                st = einsum_launch(spec, in0, o.dw[0], o.dw[1], o.act, out);
            }
            break;
        }
        case OpKind::Embedding:
            st = fdx_embedding_f32(in0, (int64_t)B * (*is)[0], o.dw[0], o.input_dim, o.output_dim, out, m.err_flag);
            break;
        case OpKind::MHA: {
            const Shape& qs = p.shapes[o.in[0]];
            const Shape& vs = p.shapes[o.in[1]];
            const int T = (int)qs[0], S = (int)vs[0], D = o.d_in, H = o.heads;
            const float* xq = p.out[o.in[0]];
            const float* xv = p.out[o.in[1]];
            const float* xk = p.out[o.in.size() > 2 ? o.in[2] : o.in[1]];
            const int64_t nk = (int64_t)H * o.dk, nv = (int64_t)H * o.dv;
            const std::vector<float*>& tmp = p.temps[idx];
            float *q = tmp[0], *k = tmp[1], *v = tmp[2], *merged = tmp[3], *scratch = tmp[4];
            if (o.dw.size() > 11 && o.dw[10]) {
                const int64_t nt = 2 * nk + nv;
                if (o.ln_src >= 0 && p.ln_fold_on[idx])
                    st = gemm_ln_launch(p.out[m.ops[o.ln_src].in[0]], (int64_t)B * T, D, o.dw[12], o.dw[13], o.dw[14], o.ln_eps, nullptr, nullptr, q,
                        (int)nt);
                else
                    st = fdx_gemm_bias_act_f32(xq, D, o.dw[10], D, B * T, (int)nt, D, 1.f, o.dw[11], 0, nullptr, nullptr, q, nt, nullptr);
                if (st != FDX_OK)
                    return st;
                if ((st = mha_prefill_strided(q, nt, T * nt, q + nk, nt, T * nt, q + 2 * nk, nt, T * nt, B, T, S, H, o.dk, o.dv, 0, merged,
                         nv, T * nv, scratch)) != FDX_OK)
                    return st;
            } else {
                if ((st = fdx_gemm_bias_act_f32(xq, D, o.dw[0], D, B * T, (int)nk, D, 1.f, o.dw[1], 0, nullptr, nullptr, q, nk, nullptr)) != FDX_OK)
                    return st;
                if ((st = fdx_gemm_bias_act_f32(xk, D, o.dw[2], D, B * S, (int)nk, D, 1.f, o.dw[3], 0, nullptr, nullptr, k, nk, nullptr)) != FDX_OK)
                    return st;
                if ((st = fdx_gemm_bias_act_f32(xv, D, o.dw[4], D, B * S, (int)nv, D, 1.f, o.dw[5], 0, nullptr, nullptr, v, nv, nullptr)) != FDX_OK)
                    return st;
                if ((st = fdx_mha_prefill_f32(q, k, v, B, T, S, H, o.dk, o.dv, 0, merged, scratch)) != FDX_OK)
                    return st;
            }
            if (o.gate) { // attention output times sigmoid(gate projection of the query) (group_query_attention_layer.hpp:157-164)
                float* gbuf = tmp[5];
                const fdx_act sg = { FDX_ACT_SIGMOID, 0.f, 0.f, 0.f };
                const size_t n = (size_t)B * (size_t)T * (size_t)nv;
                int64_t flat[5] = { 1, 1, 1, 1, (int64_t)n };
                if ((st = fdx_gemm_bias_act_f32(xq, D, o.dw[8], D, B * T, (int)nv, D, 1.f, o.dw[9], 0, nullptr, nullptr, gbuf, nv, nullptr)) != FDX_OK
                    || (st = fdx_activation_f32(gbuf, n, &sg, gbuf)) != FDX_OK
                    || (st = fdx_broadcast_combine_f32(FDX_COMBINE_MUL, merged, flat, gbuf, flat, 0, 1, 1.0f, nullptr, merged, nullptr)) != FDX_OK)
                    return st;
            }
            st = fdx_gemm_bias_act_f32(merged, nv, o.dw[6], nv, B * T, o.dout, (int)nv, 1.f, o.dw[7], 0, res, actp, out,
                o.dout, nullptr);
            break;
        }
        }
        if (st != FDX_OK)
            return st;
        if (o.softmax) // fused "softmax" activation of a conv / dense layer, in place
            st = fdx_softmax_f32(out, (int64_t)B * volume(os) / os.back(), (int)os.back(), 0, 0, out);
        return st;
    }

    std::string shape_str(const Shape& s)
    {
        std::string r = "(";
        for (size_t i = 0; i < s.size(); ++i)
            r += (i ? ", " : "") + (s[i] < 0 ? std::string("None") : std::to_string(s[i]));
        return r + ")";
    }

    fdx_status shapes_from_args(const fdx_model& m, const int64_t* in_dims, const int* in_ranks, std::vector<Shape>& shapes)
    {
        shapes.clear();
        for (size_t i = 0; i < m.inputs.size(); ++i) {
            const int rank = in_ranks[i];
            FDX_REQUIRE(rank >= 1 && rank <= 5, "input %zu: rank must be 1..5", i);
            Shape s(in_dims + i * 5 + (5 - rank), in_dims + i * 5 + 5);
            // rank and every fixed dimension must match (model.hpp:134-139, tensor_shape.hpp:246-250)
            const Shape& d = m.in_decl[i];
            bool ok = d.size() == s.size();
            for (size_t k = 0; ok && k < s.size(); ++k)
                ok = s[k] > 0 && (d[k] < 0 || d[k] == s[k]);
            if (!ok) {
                std::string want, got;
                for (const auto& ds : m.in_decl)
                    want += shape_str(ds);
                set_error("Invalid inputs shape.\nThe model takes %s but input %zu has shape %s", want.c_str(), i,
                    shape_str(s).c_str());
                return FDX_ERR_INVALID;
            }
            shapes.push_back(std::move(s));
        }
        return FDX_OK;
    }

    void write_out_shapes(const fdx_model& m, const Plan& p, int64_t* out_dims, int* out_ranks)
    {
        for (size_t i = 0; i < m.outputs.size(); ++i) {
            const Shape& s = p.shapes[m.outputs[i]];
            if (out_ranks)
                out_ranks[i] = (int)s.size();
            if (out_dims) {
                for (int k = 0; k < 5; ++k)
                    out_dims[i * 5 + k] = 1;
                for (size_t k = 0; k < s.size(); ++k)
                    out_dims[i * 5 + 5 - s.size() + k] = s[k];
            }
        }
    }

    // The depthwise 3x3 convolution in front of 1x1 convolution `idx` and that convolution as one launch.
    fdx_status run_dw_fused(fdx_model& m, Plan& p, int idx)
    {
        const Op& c = m.ops[idx];
        const Op& d = m.ops[c.fuse_dw];
        const Shape& is = p.shapes[d.in[0]];
        if (is.size() != 3)
            return FDX_ERR_UNSUPPORTED;
        const int h = (int)is[0], w = (int)is[1], ch = (int)is[2];
        int g[6];
        fdx_status st = window(h, w, d, true, g);
        if (st != FDX_OK)
            return st;
        const fdx_act a1 = to_c(d.act), a2 = to_c(c.act);
        return fdx_dwconv_pointwise_nhwc_f32(p.out[d.in[0]], p.batch, h, w, ch, d.dw[0], d.dw[1], d.sy, g[0] + d.zp[0], g[2] + d.zp[2],
            g[4], g[5], d.act.kind == FDX_ACT_NONE ? nullptr : &a1, c.dw[0], c.dw[1], c.cout,
            c.residual >= 0 ? p.out[c.residual] : nullptr, c.act.kind == FDX_ACT_NONE ? nullptr : &a2, p.out[idx]);
    }

    // Expansion, depthwise 3x3 convolution and 1x1 convolution `idx` as one launch.
    fdx_status run_block_fused(fdx_model& m, Plan& p, int idx)
    {
        const Op& c = m.ops[idx];
        const Op& d = m.ops[c.fuse_dw];
        const Op& e = m.ops[c.fuse_exp];
        const Shape& is = p.shapes[e.in[0]];
        if (is.size() != 3)
            return FDX_ERR_UNSUPPORTED;
        int h = (int)is[0], w = (int)is[1];
        const int cin = (int)is[2];
        int g[6];
        fdx_status st;
        const fdx_act a0 = to_c(e.act), a1 = to_c(d.act), a2 = to_c(c.act);
        if (e.kh != 1 || e.sy != 1) { // a small convolution on the image in place of the 1x1 expansion
            int ge[6];
            if ((st = window(h, w, e, true, ge)) != FDX_OK)
                return st;
            const int ih = h, iw = w;
            h = ge[4];
            w = ge[5];
            if ((st = window(h, w, d, true, g)) != FDX_OK)
                return st;
            return fdx_stem_block_nhwc_f32(p.out[e.in[0]], p.batch, ih, iw, cin, e.dw[0], e.dw[1], e.act.kind == FDX_ACT_NONE ? nullptr : &a0,
                e.cout, e.kh, e.sy, ge[0] + e.zp[0], ge[2] + e.zp[2], h, w, d.dw[0], d.dw[1], d.sy, g[0] + d.zp[0], g[2] + d.zp[2], g[4], g[5],
                d.act.kind == FDX_ACT_NONE ? nullptr : &a1, c.dw[0], c.dw[1], c.cout, c.residual >= 0 ? p.out[c.residual] : nullptr,
                c.act.kind == FDX_ACT_NONE ? nullptr : &a2, p.out[idx]);
        }
        st = window(h, w, d, true, g);
        if (st != FDX_OK)
            return st;
        return fdx_inverted_residual_nhwc_f32(p.out[e.in[0]], p.batch, h, w, cin, e.dw[0], e.dw[1], e.act.kind == FDX_ACT_NONE ? nullptr : &a0,
            e.cout, d.dw[0], d.dw[1], d.sy, g[0] + d.zp[0], g[2] + d.zp[2], g[4], g[5], d.act.kind == FDX_ACT_NONE ? nullptr : &a1, c.dw[0],
            c.dw[1], c.cout, c.residual >= 0 ? p.out[c.residual] : nullptr, c.act.kind == FDX_ACT_NONE ? nullptr : &a2, p.out[idx]);
    }

    // One of the three forms of a block that ends in 1x1 convolution `idx`: 3 = expansion + depthwise + projection as one
    // launch, 1 = (expansion,) depthwise + projection as one launch, 2 = a launch per layer.  A form the launchers do not
    // take falls back to the next; p.dw_fused[idx] is left at the form that ran.
    fdx_status run_block_form(fdx_model& m, Plan& p, int idx, int form)
    {
        const Op& c = m.ops[idx];
        fdx_status st = FDX_OK;
        if (form == 3 && c.fuse_exp >= 0) {
            st = run_block_fused(m, p, idx);
            if (st != FDX_ERR_UNSUPPORTED) {
                p.dw_fused[idx] = 3;
                return st;
            }
        }
        if (form == 3)
            form = 1;
        if (c.fuse_exp >= 0 && (st = run_op(m, p, c.fuse_exp)) != FDX_OK) // the expansion was skipped in the op walk
            return st;
        if (form == 1) {
            st = run_dw_fused(m, p, idx);
            if (st != FDX_ERR_UNSUPPORTED) {
                p.dw_fused[idx] = 1;
                return st;
            }
        }
        p.dw_fused[idx] = 2;
        if ((st = run_op(m, p, c.fuse_dw)) != FDX_OK)
            return st;
        return run_op(m, p, idx);
    }

    // First execution of a plan: the forms of the block are timed on the real operands (each leaves the same result in the
    // convolution's output buffer) and the plan remembers the fastest; the choice is kept per shape in the tuner's table,
    // so that an exported table pins it too.
    fdx_status choose_dw_fusion(fdx_model& m, Plan& p, int idx)
    {
        const Op& c = m.ops[idx];
        const Op& d = m.ops[c.fuse_dw];
        TuneKey key;
        std::memset(&key, 0, sizeof key);
        {
            const Shape& is = p.shapes[d.in[0]];
            key.conv = 2;
            key.M = is.size() == 3 ? (int)is[0] : 0;
            key.Cin = is.size() == 3 ? (int)is[1] : 0;
            key.K = is.size() == 3 ? (int)is[2] : 0;
            key.N = c.cout;
            key.sy = d.sy;
            key.batch = p.batch;
            key.res = c.residual >= 0;
            key.kh = c.fuse_exp >= 0 ? (int)p.shapes[m.ops[c.fuse_exp].in[0]].back() : 0; // input channels of a whole block
        }
        int known = 0;
        const bool listed = tune_lookup(key, &known);
        if (listed || tune_frozen()) {
            // Nothing is timed and the block is not in the table: the forms that win when they are timed (MobileNetV2 at
            // batch 128: the whole block as one launch on the 112- and 56-row feature maps, depthwise + projection on
            // the 28-row ones, a launch per layer below that); a form the launchers do not cover falls back inside
            // run_block_form.
            const int by_rule = key.M >= 56 ? 3 : key.M >= 28 ? 1 : 2;
            const int form = listed ? (known == 1 || known == 3 ? known : 2) : by_rule;
            return run_block_form(m, p, idx, form);
        }
        hipEvent_t e0, e1;
        if (hipEventCreate(&e0) != hipSuccess)
            return run_block_form(m, p, idx, 2);
        if (hipEventCreate(&e1) != hipSuccess) {
            (void)hipEventDestroy(e0);
            return run_block_form(m, p, idx, 2);
        }
        const int forms[3] = { 2, 1, 3 };
        float ms[3] = { 1e30f, 1e30f, 1e30f };
        fdx_status st = FDX_OK;
        for (int f = 0; f < 3 && st == FDX_OK; ++f) {
            if (forms[f] == 3 && c.fuse_exp < 0)
                continue;
            st = run_block_form(m, p, idx, forms[f]); // warm-up; tells whether the launcher takes the shape
            if (st != FDX_OK || p.dw_fused[idx] != forms[f])
                continue;
            if (f == 0)
                tune_settle_clock([&] { return run_block_form(m, p, idx, forms[0]) == FDX_OK; });
            for (int round = 0; round < 4 && st == FDX_OK; ++round) { // the shortest of four rounds: a single one is too noisy to rank forms a few percent apart
                (void)hipEventRecord(e0, stream());
                for (int r = 0; r < 3 && st == FDX_OK; ++r)
                    st = run_block_form(m, p, idx, forms[f]);
                (void)hipEventRecord(e1, stream());
                float t = 1e30f;
                if (hipEventSynchronize(e1) == hipSuccess && hipEventElapsedTime(&t, e0, e1) == hipSuccess && t < ms[f])
                    ms[f] = t;
            }
        }
        (void)hipEventDestroy(e0);
        (void)hipEventDestroy(e1);
        tune_mark();
        if (st != FDX_OK)
            return st;
        int best = 0;
        for (int f = 1; f < 3; ++f)
            if (ms[f] < ms[best])
                best = f;
        static const bool log_picks = [] { const char* e = std::getenv("FDX_TUNE_LOG"); return e && e[0] == '1'; }();
        if (log_picks)
            std::fprintf(stderr, "[fdx tune] %s + %s: a launch per layer %.1f us, depthwise + projection %.1f us, whole block %.1f us\n",
                d.name.c_str(), c.name.c_str(), ms[0] * 1e3f / 3, ms[1] * 1e3f / 3, ms[2] * 1e3f / 3);
        st = run_block_form(m, p, idx, forms[best]); // leaves the chosen form's state (and its result) behind
        if (st == FDX_OK)
            tune_store(key, p.dw_fused[idx]);
        return st;
    }

    // runs the ops at positions [from, to) of the plan's order (to < 0: to the end)
    fdx_status execute(fdx_model& m, Plan& p, int from = 0, int to = -1)
    {
        const int end = to < 0 ? (int)p.order.size() : to;
        for (int pos = from; pos < end; ++pos) {
            const int idx = p.order[(size_t)pos];
            const Op& o = m.ops[idx];
            if (o.dead)
                continue;
            fdx_status st = FDX_OK;
            if (o.fused_into >= 0 && p.dw_fused[o.fused_into] != 2)
                continue; // absorbed by (or timed together with) the 1x1 convolution behind it
            if (o.exp_into >= 0 && (p.dw_fused[o.exp_into] == 0 || p.dw_fused[o.exp_into] == 3))
                continue; // the expansion of a block that runs as one launch, or whose forms are about to be timed
            if (o.fuse_dw >= 0 && p.dw_fused[idx] == 0)
                st = choose_dw_fusion(m, p, idx);
            else if (o.fuse_dw >= 0 && p.dw_fused[idx] == 3) {
                if (o.fuse_exp >= 0) {
                    st = run_block_fused(m, p, idx);
                    if (st == FDX_ERR_UNSUPPORTED)
                        st = run_block_form(m, p, idx, 1);
                } else { // forced by a test on a pair without an expansion in front
                    p.dw_fused[idx] = 1;
                    st = run_block_form(m, p, idx, 1);
                }
            } else if (o.fuse_dw >= 0 && p.dw_fused[idx] == 1) {
                st = run_dw_fused(m, p, idx);
                if (st == FDX_ERR_UNSUPPORTED) { // forced by a test on a pair the launcher does not take
                    p.dw_fused[idx] = 2;
                    st = run_op(m, p, m.ops[idx].fuse_dw);
                    if (st == FDX_OK)
                        st = run_op(m, p, idx);
                }
            } else
                st = run_op(m, p, idx);
            if (st != FDX_OK)
                return st;
        }
        m.last_flops = p.flops;
        return FDX_OK;
    }

    fdx_status check_embedding_flag(fdx_model& m)
    {
        if (!m.has_embedding)
            return FDX_OK;
        int flag = 0;
        FDX_HIP(hipMemcpyAsync(&flag, m.err_flag, sizeof(int), hipMemcpyDeviceToHost, stream()));
        FDX_HIP(hipStreamSynchronize(stream()));
        if (flag) {
            FDX_HIP(hipMemsetAsync(m.err_flag, 0, sizeof(int), stream()));
            set_error("vocabulary item indices must all be strictly less than the value of input_dim");
            return FDX_ERR_INVALID;
        }
        return FDX_OK;
    }

    // ---- host inputs on their way to the GPU ------------------------------------------------------------------------
    // A large host input (a batch of images: tens of MB) is not handed to one pageable hipMemcpy, which stages it through
    // the runtime's own bounce buffers on the calling thread at about half the link's rate and lets the GPU wait for all of
    // it.  It goes through two pinned buffers of the library in pieces of whole samples: a few helper threads fill one
    // buffer from the caller's memory while the DMA engine drains the other, and the first convolution of the network
    // runs on each piece as soon as its copy has landed, so that only the rest of the network waits for the last piece.
    // One stager per process; host threads that predict at the same time take turns.
    struct Segment {
        const char* src;
        char* dst;
        size_t bytes;
    };
    class Stager {
    public:
        static constexpr int kLanes = 4; // the calling thread plus three helpers (two lanes: 5 % slower, eight: no faster)
        static constexpr size_t kMinBytes = 4u << 20; // below this one plain copy is as fast
        std::mutex use; // held for a whole staged input
        char* pinned[2] = { nullptr, nullptr };
        size_t pinned_bytes = 0;
        hipStream_t copy_stream = nullptr;
        hipEvent_t drained[2] = { nullptr, nullptr }; // the copy out of pinned[i] has finished
        hipEvent_t landed[8] = {};                    // one per piece in flight; the compute stream waits on it

        fdx_status prepare(size_t piece_bytes)
        {
            if (!copy_stream) {
                FDX_HIP(hipStreamCreateWithFlags(&copy_stream, hipStreamNonBlocking));
                for (auto& e : drained)
                    FDX_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
                for (auto& e : landed)
                    FDX_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            }
            if (piece_bytes > pinned_bytes) {
                for (auto& b : pinned) {
                    if (b)
                        FDX_HIP(hipHostFree(b));
                    b = nullptr;
                    FDX_HIP(hipHostMalloc(reinterpret_cast<void**>(&b), piece_bytes, hipHostMallocDefault));
                }
                pinned_bytes = piece_bytes;
            }
            if (workers.empty())
                for (int i = 1; i < kLanes; ++i)
                    workers.emplace_back([this, i] { work(i); });
            return FDX_OK;
        }
        std::mutex out_use;         // held from the first copy into pinned_out until the caller has its results
        char* pinned_out = nullptr; // results on their way back to the caller
        size_t pinned_out_bytes = 0;
        fdx_status prepare_out(size_t bytes)
        {
            if (bytes > pinned_out_bytes) {
                if (pinned_out)
                    FDX_HIP(hipHostFree(pinned_out));
                pinned_out = nullptr;
                pinned_out_bytes = 0;
                FDX_HIP(hipHostMalloc(reinterpret_cast<void**>(&pinned_out), bytes, hipHostMallocDefault));
                pinned_out_bytes = bytes;
            }
            return FDX_OK;
        }
        // copies the segments with all lanes; returns when every byte is in place
        void gather(const std::vector<Segment>& segs)
        {
            size_t total = 0;
            for (const auto& g : segs)
                total += g.bytes;
            const size_t share = (total + kLanes - 1) / kLanes;
            std::vector<std::vector<Segment>> lanes(kLanes);
            size_t lane = 0, room = share;
            for (Segment g : segs)
                while (g.bytes > 0) {
                    const size_t take = std::min(g.bytes, room);
                    lanes[lane].push_back({ g.src, g.dst, take });
                    g.src += take; g.dst += take; g.bytes -= take; room -= take;
                    if (room == 0 && lane + 1 < (size_t)kLanes) {
                        ++lane;
                        room = share;
                    }
                }
            {
                std::lock_guard<std::mutex> lock(mu);
                for (int i = 1; i < kLanes; ++i)
                    jobs[i] = &lanes[(size_t)i];
                pending = kLanes - 1;
                ++round;
            }
            wake.notify_all();
            for (const auto& g : lanes[0])
                std::memcpy(g.dst, g.src, g.bytes);
            std::unique_lock<std::mutex> lock(mu);
            done.wait(lock, [this] { return pending == 0; });
        }
        ~Stager()
        {
            {
                std::lock_guard<std::mutex> lock(mu);
                quit = true;
            }
            wake.notify_all();
            for (auto& t : workers)
                t.join();
            // pinned buffers, stream and events live until the process ends (the runtime may be gone by now)
        }

    private:
        void work(int lane)
        {
            unsigned seen = 0;
            for (;;) {
                const std::vector<Segment>* job = nullptr;
                {
                    std::unique_lock<std::mutex> lock(mu);
                    wake.wait(lock, [&] { return quit || round != seen; });
                    if (quit)
                        return;
                    seen = round;
                    job = jobs[lane];
                }
                for (const auto& g : *job)
                    std::memcpy(g.dst, g.src, g.bytes);
                {
                    std::lock_guard<std::mutex> lock(mu);
                    if (--pending == 0)
                        done.notify_all();
                }
            }
        }
        std::vector<std::thread> workers;
        std::mutex mu;
        std::condition_variable wake, done;
        const std::vector<Segment>* jobs[kLanes] = {};
        int pending = 0;
        unsigned round = 0;
        bool quit = false;
    };
    Stager& stager()
    {
        static Stager* s = new Stager; // never destroyed: its threads sleep until the process ends
        return *s;
    }

    // How many leading ops of the plan may run piece by piece (on a range of samples at a time, all pieces of op k before
    // op k + 1 of the next piece) behind the copy of the model's only input; 0 = none.  Samples are independent in every
    // device op, so what has to hold is about buffers: pieces run piece-major, so an op of piece c + 1 must not write where
    // a result of piece c still waits for a reader behind the prefix.  Buffers are recycled by liveness, hence every prefix
    // op whose result is read behind the prefix has to own its block alone among the prefix ops.  The prefix is grown
    // until it holds about as much arithmetic as the copy takes time, and cut back until that holds.
    int chunkable_prefix(const fdx_model& m, const Plan& p, int batch)
    {
        if (m.inputs.size() != 1)
            return 0;
        const int n_pos = (int)p.order.size();
        std::vector<int> root(m.ops.size(), -1);
        for (int idx : p.order)
            root[(size_t)idx] = m.ops[(size_t)idx].kind == OpKind::View ? root[(size_t)m.ops[(size_t)idx].in[0]] : idx;
        // longest run of ops that can take a range of samples: device ops outside any fused block, every choice already made
        int longest = 0;
        double flops = 0, total = p.flops > 0 ? p.flops : 1;
        // what the pieces behind the first need to travel (55 GB/s over the link) at the rate piece-sized launches compute
        // at (75 TFLOP/s), and no more than a quarter of the model: ResNet50 b64 from host memory, prefix of 12 / 11 / 8 /
        // 7 / 6 / 5 / 2 ops: 12.9 / 13.1-13.3 / 13.6 / 13.65 / 13.55 / 13.3 / 12.85 k img/s -- a longer prefix runs more
        // of the model at a quarter of the batch than the copy can hide, a shorter one leaves the copy uncovered
        const double in_bytes = 4.0 * (double)batch * (double)volume(p.shapes[(size_t)m.inputs[0]]);
        const double enough = std::min(total / 4, in_bytes / 55e9 * 75e12);
        int wanted = -1;
        for (int pos = 0; pos < n_pos; ++pos) {
            const int idx = p.order[(size_t)pos];
            const Op& o = m.ops[(size_t)idx];
            if (o.dead) {
                longest = pos + 1;
                continue;
            }
            if (o.kind == OpKind::Host || o.kind == OpKind::MHA || o.fused_into >= 0 || o.exp_into >= 0 || o.fuse_dw >= 0 || o.fuse_exp >= 0)
                break;
            if (o.kind == OpKind::Conv2D && o.dw.size() > 4 && o.dw[4] && p.conv_form[(size_t)idx] < 0)
                break;
            bool is_output = false;
            for (int out : m.outputs)
                is_output = is_output || root[(size_t)out] == root[(size_t)idx];
            if (is_output)
                break;
            longest = pos + 1;
            flops += op_flops(o, p.shapes[(size_t)idx], p.shapes, batch);
            if (wanted < 0 && flops >= enough)
                wanted = pos + 1;
        }
        // a later op that absorbs a prefix op (blocks fused into one launch) keeps that op out of the prefix
        for (int pos = longest; pos < n_pos; ++pos) {
            const Op& o = m.ops[(size_t)p.order[(size_t)pos]];
            for (int dep : { o.fuse_dw, o.fuse_exp })
                if (dep >= 0)
                    for (int q = 0; q < longest; ++q)
                        if (p.order[(size_t)q] == dep)
                            longest = q;
        }
        int cut = wanted > 0 ? std::min(wanted, longest) : longest;
        for (; cut > 0; --cut) {
            bool ok = false; // at least one op that computes
            bool clash = false;
            for (int a = 0; a < cut && !clash; ++a) {
                const int ia = p.order[(size_t)a];
                if (m.ops[(size_t)ia].dead || m.ops[(size_t)ia].kind == OpKind::View)
                    continue;
                ok = ok || m.ops[(size_t)ia].kind != OpKind::Input;
                if (p.block_of[(size_t)ia] < 0 || p.last_use[(size_t)ia] < cut)
                    continue; // consumed inside the prefix
                for (int b = 0; b < cut; ++b) {
                    const int ib = p.order[(size_t)b];
                    if (ib != ia && !m.ops[(size_t)ib].dead && p.block_of[(size_t)ib] == p.block_of[(size_t)ia])
                        clash = true;
                }
            }
            // a pair of convolutions that one launch runs stays on one side of the cut
            for (int a = 0; a < cut && !clash; ++a) {
                const int ia = p.order[(size_t)a];
                const Op& oa = m.ops[(size_t)ia];
                if (oa.dead || oa.chain < 0 || !p.chain_on[(size_t)ia])
                    continue;
                bool inside = false;
                for (int b = a + 1; b < cut; ++b)
                    inside = inside || p.order[(size_t)b] == oa.chain;
                clash = !inside;
            }
            if (ok && !clash)
                break;
        }
        return cut;
    }

    // One host input per model input, each either one contiguous block of `batch` samples or `batch` pointers to single
    // samples; copies them to the plan's input buffers and, where the network starts with a convolution of its own
    // launch, runs the first ops of the plan piece by piece behind the copy.  *done_until receives the number of leading
    // positions of the plan's order that have been executed that way.
    fdx_status stage_host_inputs(fdx_model* m, Plan* p, int batch, const float* const* in, bool per_sample, const std::vector<Shape>& shapes,
        int* done_until)
    {
        *done_until = 0;
        size_t total = 0;
        for (size_t i = 0; i < m->inputs.size(); ++i)
            total += sizeof(float) * (size_t)batch * (size_t)volume(shapes[i]);
        if (total < Stager::kMinBytes) {
            for (size_t i = 0; i < m->inputs.size(); ++i) {
                const size_t sample = sizeof(float) * (size_t)volume(shapes[i]);
                char* dst = reinterpret_cast<char*>(p->out[m->inputs[i]]);
                if (!per_sample)
                    FDX_HIP(hipMemcpyAsync(dst, in[i], sample * (size_t)batch, hipMemcpyHostToDevice, stream()));
                else
                    for (int b = 0; b < batch; ++b)
                        FDX_HIP(hipMemcpyAsync(dst + sample * (size_t)b, in[i * (size_t)batch + (size_t)b], sample, hipMemcpyHostToDevice, stream()));
            }
            return FDX_OK;
        }
        Stager& st = stager();
        std::lock_guard<std::mutex> lock(st.use);
        static const bool no_prefix = [] { const char* e = std::getenv("FDX_STAGE_PREFIX"); return e && e[0] == '0'; }();
        const int cut = batch >= 8 && !no_prefix ? chunkable_prefix(*m, *p, batch) : 0;
        static const bool stage_log = [] { const char* e = std::getenv("FDX_STAGE_LOG"); return e && e[0] == '1'; }();
        if (stage_log)
            std::fprintf(stderr, "[fdx stage] %zu bytes, prefix of %d ops (plan has %zu)\n", total, cut, p->order.size());
        // pieces of whole samples: four per input, more where a piece would exceed 16 MB
        int piece = 0; // counted over all inputs: the two pinned buffers alternate across them
        int run_done = 0; // samples the prefix has already run on (single-input models only)
        for (size_t i = 0; i < m->inputs.size(); ++i) {
            const size_t sample = sizeof(float) * (size_t)volume(shapes[i]);
            int per_piece = std::max(1, (batch + 3) / 4);
            while (per_piece > 1 && sample * (size_t)per_piece > ((size_t)16 << 20))
                per_piece = (per_piece + 1) / 2;
            fdx_status fs = st.prepare(sample * (size_t)per_piece);
            if (fs != FDX_OK)
                return fs;
            char* dst = reinterpret_cast<char*>(p->out[m->inputs[i]]);
            for (int s0 = 0; s0 < batch; s0 += per_piece, ++piece) {
                const int count = std::min(per_piece, batch - s0);
                const int slot = piece & 1;
                if (piece >= 2)
                    FDX_HIP(hipEventSynchronize(st.drained[slot])); // the copy that last read this buffer
                std::vector<Segment> segs;
                if (!per_sample)
                    segs.push_back({ reinterpret_cast<const char*>(in[i]) + sample * (size_t)s0, st.pinned[slot], sample * (size_t)count });
                else
                    for (int b = 0; b < count; ++b)
                        segs.push_back({ reinterpret_cast<const char*>(in[i * (size_t)batch + (size_t)(s0 + b)]), st.pinned[slot] + sample * (size_t)b, sample });
                st.gather(segs);
                FDX_HIP(hipMemcpyAsync(dst + sample * (size_t)s0, st.pinned[slot], sample * (size_t)count, hipMemcpyHostToDevice, st.copy_stream));
                FDX_HIP(hipEventRecord(st.drained[slot], st.copy_stream));
                FDX_HIP(hipEventRecord(st.landed[piece & 7], st.copy_stream));
                FDX_HIP(hipStreamWaitEvent(stream(), st.landed[piece & 7], 0));
                if (cut > 0) {
                    // the first `cut` ops on the samples that have landed since they last ran: every buffer they touch is
                    // entered at the first of those samples
                    const int run_from = run_done;
                    const int run_count = s0 + count - run_done;
                    run_done = s0 + count;
                    std::vector<std::pair<int, float*>> saved;
                    for (int q = 0; q < cut; ++q) {
                        const int k = p->order[(size_t)q];
                        if (m->ops[(size_t)k].dead || !p->out[(size_t)k])
                            continue;
                        saved.emplace_back(k, p->out[(size_t)k]);
                        p->out[(size_t)k] += (size_t)run_from * (size_t)volume(p->shapes[(size_t)k]);
                    }
                    const int saved_batch = p->batch;
                    p->batch = run_count;
                    const fdx_status rs = execute(*m, *p, 0, cut);
                    p->batch = saved_batch;
                    for (auto& kv : saved)
                        p->out[(size_t)kv.first] = kv.second;
                    if (rs != FDX_OK)
                        return rs;
                }
            }
        }
        *done_until = cut;
        return FDX_OK;
    }

    fdx_status predict_impl(fdx_model* m, int batch, const float* const* in, bool in_on_device, const int64_t* in_dims,
        const int* in_ranks, float* const* out, bool out_on_device, int64_t* out_dims, int* out_ranks, bool per_sample = false)
    {
        FDX_REQUIRE(m && in && in_dims && in_ranks && out, "predict: null argument");
        FDX_REQUIRE(batch > 0, "predict: batch must be positive");
        std::lock_guard<std::mutex> lock(m->mu);
        std::vector<Shape> shapes;
        fdx_status st = shapes_from_args(*m, in_dims, in_ranks, shapes);
        if (st != FDX_OK)
            return st;
        Plan* p = nullptr;
        if ((st = get_plan(m, batch, shapes, &p)) != FDX_OK)
            return st;
        // Inputs that already lie in device memory are read where they are (16-byte aligned ones: the kernels' vector
        // loads need that): the input op and every view of it point at the caller's buffer for this call.  Nothing
        // writes an input buffer, and the plan is used under the model's lock.
        struct Restore {
            Plan* plan;
            std::vector<std::pair<int, float*>> saved;
            ~Restore()
            {
                for (auto& kv : saved)
                    plan->out[kv.first] = kv.second;
            }
        } restore{ p, {} };
        int done_until = 0;
        if (!in_on_device) {
            for (size_t i = 0; i < m->inputs.size() * (per_sample ? (size_t)batch : 1); ++i)
                FDX_REQUIRE(in[i], "predict: null input %zu", i);
            if ((st = stage_host_inputs(m, p, batch, in, per_sample, shapes, &done_until)) != FDX_OK)
                return st;
        } else
            for (size_t i = 0; i < m->inputs.size(); ++i) {
                FDX_REQUIRE(in[i], "predict: null input %zu", i);
                const size_t bytes = sizeof(float) * (size_t)batch * (size_t)volume(shapes[i]);
                if ((reinterpret_cast<uintptr_t>(in[i]) & 15) == 0) {
                    float* own = p->out[m->inputs[i]];
                    for (size_t k = 0; k < p->out.size(); ++k)
                        if (p->out[k] == own && own) {
                            restore.saved.emplace_back((int)k, own);
                            p->out[k] = const_cast<float*>(in[i]);
                        }
                    continue;
                }
                FDX_HIP(hipMemcpyAsync(p->out[m->inputs[i]], in[i], bytes, hipMemcpyDeviceToDevice, stream()));
            }
        if ((st = execute(*m, *p, done_until)) != FDX_OK)
            return st;
        // Host outputs that fit come back through a pinned buffer of the library (one asynchronous copy each, then a plain
        // memcpy once the stream has drained): a pageable device-to-host copy costs about 0.1 ms however small it is.
        size_t out_total = 0;
        for (size_t i = 0; i < m->outputs.size(); ++i) {
            FDX_REQUIRE(out[i], "predict: null output %zu", i);
            out_total += sizeof(float) * (size_t)batch * (size_t)volume(p->shapes[m->outputs[i]]);
        }
        char* bounce = nullptr;
        std::unique_lock<std::mutex> bounce_lock;
        if (!out_on_device && out_total <= ((size_t)8 << 20)) {
            Stager& sg = stager();
            bounce_lock = std::unique_lock<std::mutex>(sg.out_use);
            if (sg.prepare_out(out_total) == FDX_OK)
                bounce = sg.pinned_out;
            else
                bounce_lock.unlock();
        }
        size_t at = 0;
        for (size_t i = 0; i < m->outputs.size(); ++i) {
            const size_t bytes = sizeof(float) * (size_t)batch * (size_t)volume(p->shapes[m->outputs[i]]);
            FDX_HIP(hipMemcpyAsync(bounce ? static_cast<void*>(bounce + at) : static_cast<void*>(out[i]), p->out[m->outputs[i]], bytes,
                out_on_device ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost, stream()));
            at += bytes;
        }
        if (bounce) {
            FDX_HIP(hipStreamSynchronize(stream()));
            at = 0;
            for (size_t i = 0; i < m->outputs.size(); ++i) {
                const size_t bytes = sizeof(float) * (size_t)batch * (size_t)volume(p->shapes[m->outputs[i]]);
                std::memcpy(out[i], bounce + at, bytes);
                at += bytes;
            }
            bounce_lock.unlock();
        }
        write_out_shapes(*m, *p, out_dims, out_ranks);
        if (!out_on_device || m->has_embedding) {
            FDX_HIP(hipStreamSynchronize(stream()));
            if ((st = check_embedding_flag(*m)) != FDX_OK)
                return st;
        }
        return FDX_OK;
    }

    Shape decl_shape(const Value& v)
    {
        Shape s;
        if (!v.is_array())
            throw FormatError("shape must be an array");
        for (const auto& d : v.arr)
            s.push_back(d.is_null() ? -1 : d.integer());
        return s;
    }

    fdx_status run_embedded_tests(fdx_model* m, const Value& tests, float eps)
    {
        for (const auto& t : tests.arr) {
            const Value& ins = t.at("inputs");
            const Value& outs = t.at("outputs");
            FDX_REQUIRE(ins.is_array() && outs.is_array(), "test needs inputs and outputs");
            FDX_REQUIRE(ins.size() == m->inputs.size() && outs.size() == m->outputs.size(), "test case arity does not match the model");
            std::vector<std::vector<float>> iv, ov;
            std::vector<const float*> ip;
            std::vector<int64_t> dims(5 * ins.size(), 1);
            std::vector<int> ranks(ins.size());
            for (size_t i = 0; i < ins.size(); ++i) {
                Shape s = decl_shape(ins.arr[i].at("shape"));
                iv.push_back(decode_floats(ins.arr[i].at("values")));
                FDX_REQUIRE((int64_t)iv.back().size() == volume(s), "test input %zu: values do not fill the shape", i);
                ranks[i] = (int)s.size();
                for (size_t k = 0; k < s.size(); ++k)
                    dims[i * 5 + 5 - s.size() + k] = s[k];
            }
            for (auto& v : iv)
                ip.push_back(v.data());
            std::vector<Shape> shapes;
            fdx_status st = shapes_from_args(*m, dims.data(), ranks.data(), shapes);
            if (st != FDX_OK)
                return st;
            Plan* p = nullptr;
            {
                std::lock_guard<std::mutex> lock(m->mu);
                if ((st = get_plan(m, 1, shapes, &p)) != FDX_OK)
                    return st;
                ov.resize(outs.size());
                for (size_t i = 0; i < outs.size(); ++i)
                    ov[i].resize((size_t)volume(p->shapes[m->outputs[i]]));
            }
            std::vector<float*> op;
            for (auto& v : ov)
                op.push_back(v.data());
            if ((st = predict_impl(m, 1, ip.data(), false, dims.data(), ranks.data(), op.data(), false, nullptr, nullptr)) != FDX_OK)
                return st;
            // import_model.hpp:1990-2021: absolute tolerance, NaN == NaN passes
            for (size_t i = 0; i < outs.size(); ++i) {
                std::vector<float> want = decode_floats(outs.arr[i].at("values"));
                FDX_REQUIRE(want.size() == ov[i].size(), "test failed: output %zu has %zu values, the file holds %zu", i, ov[i].size(),
                    want.size());
                for (size_t k = 0; k < want.size(); ++k) {
                    const float a = ov[i][k], b = want[k];
                    if (!(std::fabs(a - b) <= eps || (std::isnan(a) && std::isnan(b)))) {
                        set_error("test failed: output=%zu pos=%zu value=%.9g target=%.9g", i, k, a, b);
                        return FDX_ERR_INVALID;
                    }
                }
            }
        }
        return FDX_OK;
    }

} // namespace
} // namespace fdx

fdx_model::~fdx_model()
{
    if (!device_allocs.empty() || err_flag || !plans.empty()) // a model that was only checked never reached the device
        (void)hipStreamSynchronize(fdx::stream());
    for (auto& hl : host_layers)
        if (hl.vt.destroy && hl.instance)
            hl.vt.destroy(hl.instance);
    plans.clear();
    for (float* p : device_allocs)
        (void)hipFree(p);
    if (err_flag)
        (void)hipFree(err_flag);
}

extern "C" fdx_status fdx_model_create(const char* json_text, size_t len, int verify, float verify_epsilon, fdx_model** out)
{
    return fdx_model_create_custom(json_text, len, verify, verify_epsilon, nullptr, 0, out);
}

namespace fdx {
namespace {
    // Host half of loading: text -> op list -> load-time fusion.  Touches no device; throws FormatError / Unsupported.
    const Value& parse_and_build(const char* json_text, size_t len, const fdx_custom_layer* custom_layers, int n_custom_layers,
        fdx_model& model, std::unique_ptr<Value>& root_holder)
    {
        fdx_model* m = &model;
        json::Parser parser(json_text, len);
        root_holder.reset(new Value(parser.parse()));
        const Value& root = *root_holder;
        const Value* fmt = root.find("image_data_format");
        if (!fmt || !fmt->is_string() || fmt->str() != "channels_last")
            throw FormatError("only channels_last data format supported");
        const Value& arch = root.at("architecture");
        const Value& cfg = arch.at("config");
        m->name = cfg.at("name").str();
        if (const Value* h = root.find("hash"))
            if (h->is_string())
                m->hash = h->str();
        const Value& layers = cfg.at("layers");
        if (!layers.is_array())
            throw FormatError("missing layers array");
        static const Value empty_params = [] { Value v; v.type = Value::Object; return v; }();
        const Value* tp = root.find("trainable_params");
        Builder b { *m, tp ? *tp : empty_params, {} };
        b.customs = custom_layers;
        b.n_customs = n_custom_layers;
        b.scopes.emplace_back(new Scope);
        Scope& top = *b.scopes.back();
        Builder::index_layers(top, layers);
        for (const auto& s : root.at("input_shapes").arr)
            m->in_decl.push_back(decl_shape(s));
        for (const auto& s : root.at("output_shapes").arr)
            m->out_decl.push_back(decl_shape(s));
        const auto ins = model_connections(cfg.at("input_layers"));
        const auto outs = model_connections(cfg.at("output_layers"));
        if (ins.size() != m->in_decl.size())
            throw FormatError("input_shapes does not match input_layers");
        for (size_t i = 0; i < ins.size(); ++i) {
            auto lit = top.layers.find(ins[i].layer);
            if (lit == top.layers.end() || lit->second->at("class_name").str() != "InputLayer")
                throw FormatError("input_layers must name InputLayer layers");
            const Value* nodes = lit->second->find("inbound_nodes");
            if (nodes && nodes->size() != 0)
                throw FormatError("input layer is not allowed to have inbound nodes");
            Op op;
            op.kind = OpKind::Input;
            op.name = ins[i].layer;
            op.cls = "InputLayer";
            op.input_index = (int)i;
            m->ops.push_back(std::move(op));
            m->inputs.push_back((int)m->ops.size() - 1);
            top.input_ops[ins[i].layer] = m->inputs.back();
        }
        for (const auto& o : outs)
            m->outputs.push_back(b.build(top, o));
        fuse(*m);
        return root;
    }
} // namespace
} // namespace fdx

extern "C" fdx_status fdx_model_create_custom(const char* json_text, size_t len, int verify, float verify_epsilon,
    const fdx_custom_layer* custom_layers, int n_custom_layers, fdx_model** out)
{
    FDX_REQUIRE(json_text && out, "model_create: null argument");
    FDX_REQUIRE(n_custom_layers >= 0 && (n_custom_layers == 0 || custom_layers), "model_create: bad custom layer list");
    *out = nullptr;
    if (fdx_sync() != FDX_OK)
        return FDX_ERR_HIP;
    std::unique_ptr<fdx_model> m(new fdx_model);
    try {
        std::unique_ptr<Value> holder;
        const Value& root = parse_and_build(json_text, len, custom_layers, n_custom_layers, *m, holder);
        fdx_status st = upload(*m);
        if (st != FDX_OK)
            return st;
        const Value* tests = root.find("tests");
        if (verify && tests && tests->is_array()) {
            st = run_embedded_tests(m.get(), *tests, verify_epsilon);
            if (st != FDX_OK)
                return st;
        }
    } catch (const Unsupported& e) {
        set_error("%s", e.what());
        return FDX_ERR_UNSUPPORTED;
    } catch (const std::exception& e) {
        set_error("%s", e.what());
        return FDX_ERR_FORMAT;
    }
    *out = m.release();
    return FDX_OK;
}

// The host half of fdx_model_create alone: parses the text, builds and fuses the op list, decodes every parameter array
// and the embedded test tensors, and infers all shapes with unknown extents set to `unknown_extent`.  No device is
// touched, so a file can be checked where there is no GPU; the status and message are the ones fdx_model_create would
// give for the same defect.
extern "C" fdx_status fdx_model_check(const char* json_text, size_t len, int64_t unknown_extent)
{
    FDX_REQUIRE(json_text, "model_check: null argument");
    FDX_REQUIRE(unknown_extent > 0, "model_check: the stand-in for unknown extents must be positive");
    fdx_model m;
    try {
        std::unique_ptr<Value> holder;
        const Value& root = parse_and_build(json_text, len, nullptr, 0, m, holder);
        std::vector<Shape> shapes;
        for (const Shape& d : m.in_decl) {
            Shape s = d;
            for (auto& e : s)
                if (e < 0)
                    e = unknown_extent;
            shapes.push_back(s);
        }
        std::vector<Shape> all;
        const fdx_status st = infer_shapes(m, shapes, all, topo_order(m));
        if (st != FDX_OK)
            return st;
        if (const Value* tests = root.find("tests"))
            if (tests->is_array())
                for (const auto& t : tests->arr) {
                    const Value& ins = t.at("inputs");
                    const Value& outs = t.at("outputs");
                    FDX_REQUIRE(ins.is_array() && outs.is_array(), "test needs inputs and outputs");
                    FDX_REQUIRE(ins.size() == m.inputs.size() && outs.size() == m.outputs.size(), "test case arity does not match the model");
                    for (const Value* side : { &ins, &outs })
                        for (const auto& tv : side->arr) {
                            const Shape s = decl_shape(tv.at("shape"));
                            const std::vector<float> vals = decode_floats(tv.at("values"));
                            FDX_REQUIRE((int64_t)vals.size() == volume(s), "test tensor: values do not fill the shape");
                        }
                }
    } catch (const Unsupported& e) {
        set_error("%s", e.what());
        return FDX_ERR_UNSUPPORTED;
    } catch (const std::exception& e) {
        set_error("%s", e.what());
        return FDX_ERR_FORMAT;
    }
    return FDX_OK;
}

extern "C" fdx_status fdx_model_destroy(fdx_model* m)
{
    delete m;
    return FDX_OK;
}

extern "C" fdx_status fdx_model_name(const fdx_model* m, const char** name, const char** hash)
{
    FDX_REQUIRE(m, "model_name: null model");
    if (name) *name = m->name.c_str();
    if (hash) *hash = m->hash.c_str();
    return FDX_OK;
}

extern "C" fdx_status fdx_model_io_count(const fdx_model* m, int* n_inputs, int* n_outputs)
{
    FDX_REQUIRE(m, "model_io_count: null model");
    if (n_inputs) *n_inputs = (int)m->inputs.size();
    if (n_outputs) *n_outputs = (int)m->outputs.size();
    return FDX_OK;
}

extern "C" fdx_status fdx_model_io_shape(const fdx_model* m, int is_output, int index, int* rank, int64_t* dims5)
{
    FDX_REQUIRE(m && rank && dims5, "model_io_shape: null argument");
    const auto& decl = is_output ? m->out_decl : m->in_decl;
    FDX_REQUIRE(index >= 0 && index < (int)decl.size(), "model_io_shape: index out of range");
    const Shape& s = decl[index];
    *rank = (int)s.size();
    for (int k = 0; k < 5; ++k)
        dims5[k] = 1;
    for (size_t k = 0; k < s.size(); ++k)
        dims5[5 - s.size() + k] = s[k];
    return FDX_OK;
}

extern "C" fdx_status fdx_model_predict(fdx_model* m, int batch, const float* const* in, const int64_t* in_dims,
    const int* in_ranks, float* const* out, int64_t* out_dims, int* out_ranks)
{
    return predict_impl(m, batch, in, false, in_dims, in_ranks, out, false, out_dims, out_ranks);
}

extern "C" fdx_status fdx_model_predict_samples(fdx_model* m, int batch, const float* const* in_samples, const int64_t* in_dims,
    const int* in_ranks, float* const* out, int64_t* out_dims, int* out_ranks)
{
    return predict_impl(m, batch, in_samples, false, in_dims, in_ranks, out, false, out_dims, out_ranks, true);
}

extern "C" fdx_status fdx_model_predict_dev(fdx_model* m, int batch, const float* const* in_dev, const int64_t* in_dims,
    const int* in_ranks, float* const* out_dev, int64_t* out_dims, int* out_ranks)
{
    return predict_impl(m, batch, in_dev, true, in_dims, in_ranks, out_dev, true, out_dims, out_ranks);
}

extern "C" fdx_status fdx_model_infer_shapes(fdx_model* m, const int64_t* in_dims, const int* in_ranks, int64_t* out_dims,
    int* out_ranks)
{
    FDX_REQUIRE(m && in_dims && in_ranks, "infer_shapes: null argument");
    std::lock_guard<std::mutex> lock(m->mu);
    std::vector<Shape> shapes;
    fdx_status st = shapes_from_args(*m, in_dims, in_ranks, shapes);
    if (st != FDX_OK)
        return st;
    Plan tmp;
    tmp.order = topo_order(*m);
    if ((st = infer_shapes(*m, shapes, tmp.shapes, tmp.order)) != FDX_OK)
        return st;
    write_out_shapes(*m, tmp, out_dims, out_ranks);
    return FDX_OK;
}

extern "C" fdx_status fdx_model_last_flops(const fdx_model* m, double* flops)
{
    FDX_REQUIRE(m && flops, "last_flops: null argument");
    *flops = m->last_flops;
    return FDX_OK;
}

// frugally-deep's public C++ surface on top of the fdx C ABI (include/fdx.h, libfdx.so).
//
// A program written against the reference's fdeep::load_model / model::predict /
// predict_multi / fdeep::tensor API compiles against this header unchanged and runs its
// forward passes on the GPU; there is no CPU path behind it.  Interfaces mirrored:
//   tensor_shape            include/fdeep/tensor_shape.hpp:24-174
//   tensor_shape_variable   include/fdeep/tensor_shape_variable.hpp:20-105
//   tensor_pos              include/fdeep/tensor_pos.hpp:18-114
//   tensor, tensors         include/fdeep/tensor.hpp:28-168
//   show_* / *_bytes        include/fdeep/tensor.hpp:1203-1280, tensor_shape.hpp:357-373
//   model, load_model, read_model, read_model_from_string, loggers
//                           include/fdeep/model.hpp:20-301
// Errors are std::runtime_error, as raised by include/fdeep/common.hpp:42-57.
// Custom layer creators (import_model.hpp:374-381): supported through internal::layer_creators below; such
// layers run on the host between device segments.  A layer type nobody knows fails at load with the
// reference's "unknown layer type: X" message.
#pragma once

#include <algorithm>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <fstream>
#include <functional>
#include <iostream>
#include <iterator>
#include <map>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "../fdx.h"

namespace fdeep {

using float_type = float;
using float_vec = std::vector<float_type>;
using shared_float_vec = std::shared_ptr<float_vec>;

namespace internal {
    inline void raise_error(const std::string& msg) { throw std::runtime_error(msg); }
    inline void assertion(bool cond, const std::string& msg)
    {
        if (!cond)
            raise_error(msg);
    }
    inline void check(fdx_status st)
    {
        if (st != FDX_OK)
            raise_error(fdx_last_error());
    }
}

class tensor_shape {
public:
    explicit tensor_shape(std::size_t depth)
        : rank_(1), size_dim_5_(1), size_dim_4_(1), height_(1), width_(1), depth_(depth) {}
    tensor_shape(std::size_t width, std::size_t depth)
        : rank_(2), size_dim_5_(1), size_dim_4_(1), height_(1), width_(width), depth_(depth) {}
    tensor_shape(std::size_t height, std::size_t width, std::size_t depth)
        : rank_(3), size_dim_5_(1), size_dim_4_(1), height_(height), width_(width), depth_(depth) {}
    tensor_shape(std::size_t size_dim_4, std::size_t height, std::size_t width, std::size_t depth)
        : rank_(4), size_dim_5_(1), size_dim_4_(size_dim_4), height_(height), width_(width), depth_(depth) {}
    tensor_shape(std::size_t size_dim_5, std::size_t size_dim_4, std::size_t height, std::size_t width, std::size_t depth)
        : rank_(5), size_dim_5_(size_dim_5), size_dim_4_(size_dim_4), height_(height), width_(width), depth_(depth) {}

    std::size_t volume() const { return size_dim_5_ * size_dim_4_ * height_ * width_ * depth_; }
    std::size_t rank() const { return rank_; }
    std::size_t minimal_rank() const
    {
        if (size_dim_5_ > 1) return 5;
        if (size_dim_4_ > 1) return 4;
        if (height_ > 1) return 3;
        if (width_ > 1) return 2;
        return 1;
    }
    void shrink_rank() { rank_ = minimal_rank(); }
    // include/fdeep/tensor_shape.hpp:143-146
    void shrink_rank_with_min(std::size_t min_rank_to_keep) { rank_ = std::max(minimal_rank(), min_rank_to_keep); }
    void maximize_rank() { rank_ = 5; }
    // the extents the rank covers, outermost first (include/fdeep/tensor_shape.hpp:153-164)
    std::vector<std::size_t> dimensions() const
    {
        const std::vector<std::size_t> all = dimensions5();
        return std::vector<std::size_t>(all.end() - static_cast<std::ptrdiff_t>(rank_), all.end());
    }
    // all five right-aligned extents
    std::vector<std::size_t> dimensions5() const { return { size_dim_5_, size_dim_4_, height_, width_, depth_ }; }

    std::size_t rank_;
    std::size_t size_dim_5_;
    std::size_t size_dim_4_;
    std::size_t height_;
    std::size_t width_;
    std::size_t depth_;
};

inline bool operator==(const tensor_shape& a, const tensor_shape& b)
{
    return a.rank() == b.rank() && a.dimensions5() == b.dimensions5();
}
inline bool operator!=(const tensor_shape& a, const tensor_shape& b) { return !(a == b); }

inline tensor_shape create_tensor_shape_from_dims(const std::vector<std::size_t>& dims)
{
    internal::assertion(dims.size() >= 1 && dims.size() <= 5, "Invalid number of dimensions");
    switch (dims.size()) {
    case 1: return tensor_shape(dims[0]);
    case 2: return tensor_shape(dims[0], dims[1]);
    case 3: return tensor_shape(dims[0], dims[1], dims[2]);
    case 4: return tensor_shape(dims[0], dims[1], dims[2], dims[3]);
    default: return tensor_shape(dims[0], dims[1], dims[2], dims[3], dims[4]);
    }
}

inline std::string show_tensor_shape(const tensor_shape& s)
{
    const auto d = s.dimensions5();
    std::string r = std::to_string(s.rank()) + "(";
    for (std::size_t i = 5 - s.rank(); i < 5; ++i)
        r += std::to_string(d[i]) + (i + 1 < 5 ? ", " : "");
    return r + ")";
}
inline std::string show_tensor_shapes(const std::vector<tensor_shape>& shapes)
{
    std::string r = "[";
    for (std::size_t i = 0; i < shapes.size(); ++i)
        r += (i ? ", " : "") + show_tensor_shape(shapes[i]);
    return r + "]";
}

// A shape whose dimensions may be unknown until predict time (a null in the file).
class tensor_shape_variable {
public:
    tensor_shape_variable(std::size_t rank, const std::vector<std::int64_t>& dims5)
        : rank_(rank), dims_(dims5) {}
    std::size_t rank() const { return rank_; }
    // product of the known extents, unknown ones counting as 1 (include/fdeep/tensor_shape_variable.hpp:87-90)
    std::size_t minimal_volume() const
    {
        std::size_t v = 1;
        for (std::int64_t d : dims_)
            v *= d >= 0 ? static_cast<std::size_t>(d) : 1;
        return v;
    }
    bool fixed(std::size_t i) const { return dims_[i] >= 0; }     // i indexes the 5 right-aligned dims
    std::int64_t dim(std::size_t i) const { return dims_[i]; }
    std::size_t rank_;
    std::vector<std::int64_t> dims_; // size_dim_5, size_dim_4, height, width, depth; -1 = variable
};

inline std::string show_tensor_shape_variable(const tensor_shape_variable& s)
{
    std::string r = std::to_string(s.rank()) + "(";
    for (std::size_t i = 5 - s.rank(); i < 5; ++i)
        r += (s.fixed(i) ? std::to_string(s.dim(i)) : std::string("None")) + (i + 1 < 5 ? ", " : "");
    return r + ")";
}
inline std::string show_tensor_shapes_variable(const std::vector<tensor_shape_variable>& shapes)
{
    std::string r = "[";
    for (std::size_t i = 0; i < shapes.size(); ++i)
        r += (i ? ", " : "") + show_tensor_shape_variable(shapes[i]);
    return r + "]";
}

namespace internal {
    // fills unknown dimensions from `def`, right-aligned (include/fdeep/tensor_shape.hpp, make_tensor_shape_with)
    inline tensor_shape make_tensor_shape_with(const tensor_shape& def, const tensor_shape_variable& s)
    {
        const auto dd = def.dimensions5();
        std::vector<std::size_t> dims;
        for (std::size_t i = 5 - s.rank(); i < 5; ++i)
            dims.push_back(s.fixed(i) ? static_cast<std::size_t>(s.dim(i)) : dd[i]);
        return create_tensor_shape_from_dims(dims);
    }
}

class tensor_pos {
public:
    explicit tensor_pos(std::size_t z)
        : rank_(1), pos_dim_5_(0), pos_dim_4_(0), y_(0), x_(0), z_(z) {}
    tensor_pos(std::size_t x, std::size_t z)
        : rank_(2), pos_dim_5_(0), pos_dim_4_(0), y_(0), x_(x), z_(z) {}
    tensor_pos(std::size_t y, std::size_t x, std::size_t z)
        : rank_(3), pos_dim_5_(0), pos_dim_4_(0), y_(y), x_(x), z_(z) {}
    tensor_pos(std::size_t pos_dim_4, std::size_t y, std::size_t x, std::size_t z)
        : rank_(4), pos_dim_5_(0), pos_dim_4_(pos_dim_4), y_(y), x_(x), z_(z) {}
    tensor_pos(std::size_t pos_dim_5, std::size_t pos_dim_4, std::size_t y, std::size_t x, std::size_t z)
        : rank_(5), pos_dim_5_(pos_dim_5), pos_dim_4_(pos_dim_4), y_(y), x_(x), z_(z) {}
    std::size_t rank() const { return rank_; }
    // the coordinates the rank covers, outermost first (include/fdeep/tensor_pos.hpp)
    std::vector<std::size_t> dimensions() const
    {
        const std::vector<std::size_t> all = { pos_dim_5_, pos_dim_4_, y_, x_, z_ };
        return std::vector<std::size_t>(all.end() - static_cast<std::ptrdiff_t>(rank_), all.end());
    }
    std::size_t rank_;
    std::size_t pos_dim_5_;
    std::size_t pos_dim_4_;
    std::size_t y_;
    std::size_t x_;
    std::size_t z_;
};

// include/fdeep/tensor_pos.hpp:116-147
inline tensor_pos create_tensor_pos_from_dims(const std::vector<std::size_t>& dimensions)
{
    internal::assertion(dimensions.size() >= 1 && dimensions.size() <= 5, "Invalid tensor-pos dimensions");
    switch (dimensions.size()) {
    case 1: return tensor_pos(dimensions[0]);
    case 2: return tensor_pos(dimensions[0], dimensions[1]);
    case 3: return tensor_pos(dimensions[0], dimensions[1], dimensions[2]);
    case 4: return tensor_pos(dimensions[0], dimensions[1], dimensions[2], dimensions[3]);
    default: return tensor_pos(dimensions[0], dimensions[1], dimensions[2], dimensions[3], dimensions[4]);
    }
}

// Rank <= 5, right-aligned, row-major, channels-last fp32 values on a shared buffer:
// copying a tensor shares the buffer.
class tensor {
public:
    tensor(const tensor_shape& shape, const shared_float_vec& values)
        : shape_(shape), values_(values)
    {
        internal::assertion(shape.volume() == values->size(), "invalid number of values. shape: "
                + show_tensor_shape(shape) + ", value count: " + std::to_string(values->size()));
    }
    tensor(const tensor_shape& shape, float_vec&& values)
        : tensor(shape, std::make_shared<float_vec>(std::move(values))) {}
    tensor(const tensor_shape& shape, const float_vec& values)
        : tensor(shape, std::make_shared<float_vec>(values)) {}
    tensor(const tensor_shape& shape, float_type value)
        : tensor(shape, std::make_shared<float_vec>(shape.volume(), value)) {}

    float_type get(const tensor_pos& pos) const
    {
        internal::assertion(pos.rank() == shape_.rank(), "Invalid position rank for tensor");
        return get_ignore_rank(pos);
    }
    float_type get_ignore_rank(const tensor_pos& pos) const { return (*values_)[idx_ignore_rank(pos)]; }
    const float_type& get_ref_ignore_rank(const tensor_pos& pos) const { return (*values_)[idx_ignore_rank(pos)]; }
    float_type& get_ref_ignore_rank(const tensor_pos& pos) { return (*values_)[idx_ignore_rank(pos)]; }
    // the value at a signed position, pad_value outside the tensor (include/fdeep/tensor.hpp:66-79)
    float_type get_padded(float_type pad_value, int d5, int d4, int y, int x, int z) const
    {
        if (d5 < 0 || d5 >= static_cast<int>(shape_.size_dim_5_) || d4 < 0 || d4 >= static_cast<int>(shape_.size_dim_4_) || y < 0
            || y >= static_cast<int>(shape_.height_) || x < 0 || x >= static_cast<int>(shape_.width_) || z < 0
            || z >= static_cast<int>(shape_.depth_))
            return pad_value;
        return get_ignore_rank(tensor_pos(static_cast<std::size_t>(d5), static_cast<std::size_t>(d4), static_cast<std::size_t>(y),
            static_cast<std::size_t>(x), static_cast<std::size_t>(z)));
    }
    // the five-index forms the reference keeps as deprecated (include/fdeep/tensor.hpp:95-112): rank is ignored
    float_type get(std::size_t pos_dim_5, std::size_t pos_dim_4, std::size_t y, std::size_t x, std::size_t z) const
    {
        return get_ignore_rank(tensor_pos(pos_dim_5, pos_dim_4, y, x, z));
    }
    void set(std::size_t pos_dim_5, std::size_t pos_dim_4, std::size_t y, std::size_t x, std::size_t z, float_type value)
    {
        set_ignore_rank(tensor_pos(pos_dim_5, pos_dim_4, y, x, z), value);
    }
    void set(const tensor_pos& pos, float_type value)
    {
        internal::assertion(pos.rank() == shape_.rank(), "Invalid position rank for tensor");
        set_ignore_rank(pos, value);
    }
    void set_ignore_rank(const tensor_pos& pos, float_type value) { (*values_)[idx_ignore_rank(pos)] = value; }
    const tensor_shape& shape() const { return shape_; }
    void shrink_rank() { shape_.shrink_rank(); }
    void shrink_rank_with_min(std::size_t min_rank_to_keep) { shape_.shrink_rank_with_min(min_rank_to_keep); }
    void maximize_rank() { shape_.maximize_rank(); }
    std::size_t depth() const { return shape_.depth_; }
    std::size_t height() const { return shape_.height_; }
    std::size_t width() const { return shape_.width_; }
    std::size_t rank() const { return shape_.rank(); }
    const shared_float_vec& as_vector() const { return values_; }
    shared_float_vec& as_vector() { return values_; }
    float_vec to_vector() const { return *values_; }

private:
    std::size_t idx_ignore_rank(const tensor_pos& p) const
    {
        return (((p.pos_dim_5_ * shape_.size_dim_4_ + p.pos_dim_4_) * shape_.height_ + p.y_) * shape_.width_ + p.x_)
            * shape_.depth_ + p.z_;
    }
    tensor_shape shape_;
    shared_float_vec values_;
};

using tensors = std::vector<tensor>;
using tensors_vec = std::vector<tensors>;

inline std::string show_tensor(const tensor& t)
{
    // every value with four decimals, padded on the left with spaces to the longest of them
    // (include/fdeep/tensor.hpp:1203-1218), nested by dim5 / dim4 / height / width / depth
    const auto& v = *t.as_vector();
    const auto& s = t.shape();
    std::vector<std::string> strs;
    strs.reserve(v.size());
    std::size_t longest = 0;
    for (float_type f : v) {
        std::ostringstream one;
        one.setf(std::ios::fixed);
        one.precision(4);
        one << f;
        strs.push_back(one.str());
        longest = std::max(longest, strs.back().size());
    }
    for (auto& str : strs)
        str.insert(0, longest - str.size(), ' ');
    std::ostringstream os;
    std::size_t i = 0;
    os << "[";
    for (std::size_t d5 = 0; d5 < s.size_dim_5_; ++d5) {
        os << (d5 ? ", [" : "[");
        for (std::size_t d4 = 0; d4 < s.size_dim_4_; ++d4) {
            os << (d4 ? ", [" : "[");
            for (std::size_t y = 0; y < s.height_; ++y) {
                os << (y ? ", [" : "[");
                for (std::size_t x = 0; x < s.width_; ++x) {
                    os << (x ? ", [" : "[");
                    for (std::size_t z = 0; z < s.depth_; ++z)
                        os << (z ? ", " : "") << strs[i++];
                    os << "]";
                }
                os << "]";
            }
            os << "]";
        }
        os << "]";
    }
    os << "]";
    return os.str();
}
inline std::string show_tensors(const tensors& ts)
{
    std::string r = "[";
    for (std::size_t i = 0; i < ts.size(); ++i)
        r += (i ? ", " : "") + show_tensor(ts[i]);
    return r + "]";
}

// 8-bit row-wise channels-last memory <-> tensor, [0,255] mapped linearly onto [low, high]
inline tensor tensor_from_bytes(const std::uint8_t* value_ptr, std::size_t height, std::size_t width,
    std::size_t channels, float_type low = 0.0f, float_type high = 1.0f)
{
    float_vec values(height * width * channels);
    for (std::size_t i = 0; i < values.size(); ++i)
        values[i] = low + (high - low) * (static_cast<float_type>(value_ptr[i]) / 255.0f);
    return tensor(tensor_shape(height, width, channels), std::move(values));
}
inline void tensor_into_bytes(const tensor& t, std::uint8_t* value_ptr, std::size_t bytes_available,
    float_type low = 0.0f, float_type high = 1.0f)
{
    const auto& values = *t.as_vector();
    internal::assertion(bytes_available == values.size(), "invalid buffer size");
    for (std::size_t i = 0; i < values.size(); ++i) {
        const float_type scaled = (values[i] - low) / (high - low) * 255.0f;
        value_ptr[i] = static_cast<std::uint8_t>(std::min(255.0f, std::max(0.0f, std::round(scaled))));
    }
}
inline std::vector<std::uint8_t> tensor_to_bytes(const tensor& t, float_type low = 0.0f, float_type high = 1.0f)
{
    std::vector<std::uint8_t> bytes(t.shape().volume(), 0);
    tensor_into_bytes(t, bytes.data(), bytes.size(), low, high);
    return bytes;
}

// All values of all tensors, in order, cut anew into vectors_size vectors of vector_size tensors of shape
// (height, width, depth) (include/fdeep/tensor.hpp:1282-1303)
inline tensors_vec reshape_tensor_vectors(std::size_t vectors_size, std::size_t vector_size, std::size_t depth, std::size_t height,
    std::size_t width, const tensors_vec& tss)
{
    float_vec values;
    for (const auto& ts : tss)
        for (const auto& t : ts)
            values.insert(values.end(), t.as_vector()->begin(), t.as_vector()->end());
    internal::assertion(values.size() == vectors_size * vector_size * height * width * depth,
        "Invalid number of values for reshape target.");
    const std::size_t per_tensor = depth * height * width;
    tensors_vec result;
    std::size_t at = 0;
    while (at < values.size()) {
        if (result.empty() || result.back().size() == vector_size)
            result.emplace_back();
        const std::size_t n = std::min(per_tensor, values.size() - at);
        result.back().push_back(tensor(tensor_shape(height, width, depth),
            float_vec(values.begin() + static_cast<std::ptrdiff_t>(at), values.begin() + static_cast<std::ptrdiff_t>(at + n))));
        at += n;
    }
    return result;
}

namespace internal {
    // Extension point for layer classes the device path does not know: a subclass of `layer` implements
    // apply_impl on host tensors and is produced by a creator registered under the Keras class name
    // (include/fdeep/layers/layer.hpp:32-88, include/fdeep/import_model.hpp:374-381).  The creator receives
    // the layer's JSON text instead of a parsed nlohmann::json object, and get_param returns the decoded
    // floats of one trainable_params entry.
    class layer {
    public:
        explicit layer(const std::string& name)
            : name_(name)
        {
        }
        virtual ~layer() = default;
        virtual tensors apply_impl(const tensors& inputs) const = 0;
        std::string name_;
    };
    using layer_ptr = std::shared_ptr<layer>;
    using get_param_f = std::function<float_vec(const std::string& layer_name, const std::string& param_name)>;
    using layer_creator = std::function<layer_ptr(const get_param_f&, const std::string& layer_json, const std::string& name)>;
    using layer_creators = std::map<std::string, layer_creator>;

    inline fdx_status custom_create(void* user, const char* layer_name, const char* config_json, std::size_t config_len,
        fdx_param_getter get_param, void* get_param_ctx, void** instance)
    {
        try {
            const auto& creator = *static_cast<const layer_creator*>(user);
            const get_param_f getter = [get_param, get_param_ctx](const std::string& l, const std::string& k) {
                const float* values = nullptr;
                std::size_t count = 0;
                check(get_param(get_param_ctx, l.c_str(), k.c_str(), &values, &count));
                return float_vec(values, values + count);
            };
            layer_ptr made = creator(getter, std::string(config_json, config_len), layer_name);
            if (!made) {
                fdx_set_last_error("custom layer creator returned no layer");
                return FDX_ERR_INVALID;
            }
            *instance = new layer_ptr(std::move(made));
            return FDX_OK;
        } catch (const std::exception& e) {
            fdx_set_last_error(e.what());
            return FDX_ERR_INVALID;
        }
    }
    inline fdx_status custom_apply(void* instance, int n_inputs, const float* const* inputs, const int* in_ranks,
        const std::int64_t* in_dims5, float* output, int* out_rank, std::int64_t* out_dims5)
    {
        try {
            tensors ins;
            for (int i = 0; i < n_inputs; ++i) {
                std::vector<std::size_t> dims;
                for (int k = 5 - in_ranks[i]; k < 5; ++k)
                    dims.push_back(static_cast<std::size_t>(in_dims5[i * 5 + k]));
                const tensor_shape shape = create_tensor_shape_from_dims(dims);
                ins.emplace_back(shape, float_vec(inputs[i], inputs[i] + shape.volume()));
            }
            const tensors outs = (*static_cast<layer_ptr*>(instance))->apply_impl(ins);
            if (outs.size() != 1) {
                fdx_set_last_error("a custom layer must return exactly one tensor");
                return FDX_ERR_INVALID;
            }
            const tensor_shape& os = outs[0].shape();
            *out_rank = static_cast<int>(os.rank());
            const auto d = os.dimensions5();
            for (std::size_t k = 0; k < 5; ++k)
                out_dims5[k] = static_cast<std::int64_t>(d[k]);
            if (output)
                std::copy(outs[0].as_vector()->begin(), outs[0].as_vector()->end(), output);
            return FDX_OK;
        } catch (const std::exception& e) {
            fdx_set_last_error(e.what());
            return FDX_ERR_INVALID;
        }
    }
    inline void custom_destroy(void* instance) { delete static_cast<layer_ptr*>(instance); }
}

inline void cout_logger(const std::string& str) { std::cout << str << std::flush; }
inline void dev_null_logger(const std::string&) {}

class model {
public:
    // One forward pass.  include/fdeep/model.hpp:23-26,132-151
    tensors predict(const tensors& inputs) const { return predict_multi({ inputs }, false).front(); }

    // Independent samples; all of them go through ONE batched launch sequence on the GPU, whatever
    // `parallelly` says (the reference starts a CPU thread per sample, model.hpp:28-42).
    std::vector<tensors> predict_multi(const std::vector<tensors>& inputs_vec, bool parallelly) const
    {
        (void)parallelly;
        if (inputs_vec.empty())
            return {};
        const std::size_t n_in = input_shapes_.size(), n_out = output_shapes_.size(), batch = inputs_vec.size();
        for (const auto& ins : inputs_vec) {
            bool ok = ins.size() == n_in;
            for (std::size_t i = 0; ok && i < n_in; ++i)
                ok = ins[i].shape() == inputs_vec.front()[i].shape();
            if (!ok)
                return predict_one_by_one(inputs_vec); // ragged shapes: still correct, one launch sequence each
        }
        // one pointer per sample and input: the library gathers them on their way to the GPU, nothing is concatenated here
        std::vector<const float*> in_ptrs(n_in * batch);
        std::vector<std::int64_t> in_dims(5 * n_in);
        std::vector<int> in_ranks(n_in);
        for (std::size_t i = 0; i < n_in; ++i) {
            const tensor_shape& s = inputs_vec.front()[i].shape();
            const auto d = s.dimensions5();
            for (int k = 0; k < 5; ++k)
                in_dims[i * 5 + k] = static_cast<std::int64_t>(d[k]);
            in_ranks[i] = static_cast<int>(s.rank());
            for (std::size_t b = 0; b < batch; ++b)
                in_ptrs[i * batch + b] = inputs_vec[b][i].as_vector()->data();
        }
        std::vector<std::int64_t> out_dims(5 * n_out);
        std::vector<int> out_ranks(n_out);
        internal::check(fdx_model_infer_shapes(handle_.get(), in_dims.data(), in_ranks.data(), out_dims.data(), out_ranks.data()));
        std::vector<float_vec> outs(n_out);
        std::vector<float*> out_ptrs(n_out);
        std::vector<tensor_shape> out_shapes;
        for (std::size_t i = 0; i < n_out; ++i) {
            std::vector<std::size_t> dims;
            for (int k = 5 - out_ranks[i]; k < 5; ++k)
                dims.push_back(static_cast<std::size_t>(out_dims[i * 5 + k]));
            out_shapes.push_back(create_tensor_shape_from_dims(dims));
            outs[i].resize(batch * out_shapes.back().volume());
            out_ptrs[i] = outs[i].data();
        }
        internal::check(fdx_model_predict_samples(handle_.get(), static_cast<int>(batch), in_ptrs.data(), in_dims.data(),
            in_ranks.data(), out_ptrs.data(), nullptr, nullptr));
        std::vector<tensors> result(batch);
        for (std::size_t b = 0; b < batch; ++b)
            for (std::size_t i = 0; i < n_out; ++i) {
                const std::size_t vol = out_shapes[i].volume();
                result[b].emplace_back(out_shapes[i],
                    float_vec(outs[i].begin() + static_cast<std::ptrdiff_t>(b * vol), outs[i].begin() + static_cast<std::ptrdiff_t>((b + 1) * vol)));
            }
        return result;
    }

    // index of the strongest output neuron of a single (1, 1, z) output; first maximum wins (tensor.hpp:281-302)
    std::size_t predict_class(const tensors& inputs) const { return predict_class_with_confidence(inputs).first; }
    std::pair<std::size_t, float_type> predict_class_with_confidence(const tensors& inputs) const
    {
        const tensors outputs = predict(inputs);
        internal::assertion(outputs.size() == 1, std::string("invalid number of outputs.\n") + "Use model::predict instead of model::predict_class.");
        const auto& s = outputs.front().shape();
        internal::assertion(s.size_dim_5_ * s.size_dim_4_ * s.height_ * s.width_ == 1,
            std::string("invalid output shape.\n") + "Use model::predict instead of model::predict_class.");
        const auto& v = *outputs.front().as_vector();
        std::size_t best = 0;
        float_type best_val = std::numeric_limits<float_type>::lowest();
        for (std::size_t i = 0; i < v.size(); ++i)
            if (v[i] > best_val) {
                best_val = v[i];
                best = i;
            }
        return { best, best_val };
    }
    float_type predict_single_output(const tensors& inputs) const
    {
        const tensors outputs = predict(inputs);
        internal::assertion(outputs.size() == 1, "invalid number of outputs.\nUse model::predict instead of model::predict_single_output.");
        internal::assertion(outputs.front().shape().volume() == 1, "invalid output shape.\nUse model::predict instead of model::predict_single_output.");
        return outputs.front().as_vector()->front();
    }

    const std::vector<tensor_shape_variable>& get_input_shapes() const { return input_shapes_; }
    const std::vector<tensor_shape_variable>& get_output_shapes() const { return output_shapes_; }
    const std::vector<tensor_shape> get_dummy_input_shapes() const
    {
        std::vector<tensor_shape> r;
        for (const auto& s : input_shapes_)
            r.push_back(internal::make_tensor_shape_with(tensor_shape(42, 42, 42), s));
        return r;
    }
    tensors generate_dummy_inputs() const
    {
        tensors r;
        for (const auto& s : get_dummy_input_shapes())
            r.emplace_back(s, 0.0f);
        return r;
    }
    // seconds for one forward pass on zero-filled dummy inputs (model.hpp:98-104)
    double test_speed() const
    {
        const auto inputs = generate_dummy_inputs();
        const auto t0 = std::chrono::steady_clock::now();
        predict(inputs);
        return std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    }
    const std::string& name() const { return name_; }
    const std::string& hash() const { return hash_; }

    // the underlying C handle, for the session (key/value cache decode) entry points of fdx.h
    fdx_model* handle() const { return handle_.get(); }

private:
    model() = default;
    std::vector<tensors> predict_one_by_one(const std::vector<tensors>& inputs_vec) const
    {
        std::vector<tensors> r;
        for (const auto& ins : inputs_vec)
            r.push_back(predict_multi({ ins }, false).front());
        return r;
    }
    friend model read_model_from_string(const std::string&, bool, const std::function<void(std::string)>&, float_type,
        const internal::layer_creators&);
    std::shared_ptr<fdx_model> handle_;
    std::vector<tensor_shape_variable> input_shapes_, output_shapes_;
    std::string name_, hash_;
};

// Loads a converted-JSON model held in memory.  include/fdeep/model.hpp:271-281 (and 198-267 for the steps logged)
inline model read_model_from_string(const std::string& content, bool verify = true,
    const std::function<void(std::string)>& logger = cout_logger, float_type verify_epsilon = static_cast<float_type>(0.0001),
    const internal::layer_creators& custom_layer_creators = internal::layer_creators())
{
    const auto log = [&logger](const std::string& msg) {
        if (logger)
            logger(msg + "\n");
    };
    const auto t0 = std::chrono::steady_clock::now();
    log(std::string("Loading json, building model and uploading weights") + (verify ? ", running embedded tests" : "") + " ... ");
    fdx_model* raw = nullptr;
    std::vector<fdx_custom_layer> customs;
    for (const auto& kv : custom_layer_creators)
        customs.push_back(fdx_custom_layer { kv.first.c_str(), &internal::custom_create, &internal::custom_apply,
            &internal::custom_destroy, const_cast<internal::layer_creator*>(&kv.second) });
    internal::check(fdx_model_create_custom(content.data(), content.size(), verify ? 1 : 0, verify_epsilon, customs.data(),
        static_cast<int>(customs.size()), &raw));
    model m;
    m.handle_ = std::shared_ptr<fdx_model>(raw, [](fdx_model* p) { fdx_model_destroy(p); });
    int n_in = 0, n_out = 0;
    internal::check(fdx_model_io_count(raw, &n_in, &n_out));
    for (int out = 0; out < 2; ++out)
        for (int i = 0; i < (out ? n_out : n_in); ++i) {
            int rank = 0;
            std::int64_t dims[5];
            internal::check(fdx_model_io_shape(raw, out, i, &rank, dims));
            (out ? m.output_shapes_ : m.input_shapes_).emplace_back(static_cast<std::size_t>(rank), std::vector<std::int64_t>(dims, dims + 5));
        }
    const char *name = nullptr, *hash = nullptr;
    internal::check(fdx_model_name(raw, &name, &hash));
    m.name_ = name;
    m.hash_ = hash;
    log("done. elapsed time: " + std::to_string(std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count()) + " s");
    return m;
}

inline model read_model(std::istream& model_file_stream, bool verify = true,
    const std::function<void(std::string)>& logger = cout_logger, float_type verify_epsilon = static_cast<float_type>(0.0001),
    const internal::layer_creators& custom_layer_creators = internal::layer_creators())
{
    const std::string content((std::istreambuf_iterator<char>(model_file_stream)), std::istreambuf_iterator<char>());
    return read_model_from_string(content, verify, logger, verify_epsilon, custom_layer_creators);
}

// include/fdeep/model.hpp:285-301
inline model load_model(const std::string& file_path, bool verify = true,
    const std::function<void(std::string)>& logger = cout_logger, float_type verify_epsilon = static_cast<float_type>(0.0001),
    const internal::layer_creators& custom_layer_creators = internal::layer_creators())
{
    std::ifstream in_stream(file_path, std::ios::binary);
    internal::assertion(in_stream.good(), "Can not open " + file_path);
    if (logger)
        logger("Loading model " + file_path + "\n");
    return read_model(in_stream, verify, logger, verify_epsilon, custom_layer_creators);
}

} // namespace fdeep

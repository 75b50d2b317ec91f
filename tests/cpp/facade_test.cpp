// Drives the C++ facade the way the reference's own doctest files drive fdeep
// (test/test_model_exhaustive_test.cpp:11-20): load a self-verifying model file with a tight
// epsilon, then predict_multi on dummy inputs serially and "in parallel"; plus the error paths a
// caller can hit.  Usage: facade_test <model.json> <expected_class_of_first_test_input>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <fdeep/fdeep.hpp>
#include <thread>

#define EXPECT(cond)                                                     \
    do {                                                                 \
        if (!(cond)) {                                                   \
            std::fprintf(stderr, "FAILED %s:%d %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                    \
        }                                                                \
    } while (0)

template <typename F>
static bool throws_with(F f, const std::string& needle)
{
    try {
        f();
    } catch (const std::runtime_error& e) {
        return std::string(e.what()).find(needle) != std::string::npos;
    }
    return false;
}

int main(int argc, char** argv)
{
    if (argc < 2)
        return 2;
    std::string log;
    const auto model = fdeep::load_model(argv[1], true, [&log](const std::string& s) { log += s; }, static_cast<fdeep::float_type>(0.00001));
    EXPECT(log.find("Loading model") != std::string::npos && log.find("done. elapsed time") != std::string::npos);
    EXPECT(model.name() == "small_cnn");
    EXPECT(model.get_input_shapes().size() == 1 && model.get_output_shapes().size() == 1);
    EXPECT(fdeep::show_tensor_shapes_variable(model.get_input_shapes()) == "[3(32, 32, 3)]");

    const auto dummy = model.generate_dummy_inputs();
    EXPECT(dummy.size() == 1 && dummy[0].shape() == fdeep::tensor_shape(32, 32, 3));
    const std::vector<fdeep::tensors> many(10, dummy);
    const auto serial = model.predict_multi(many, false);
    const auto parallel = model.predict_multi(many, true);
    EXPECT(serial.size() == 10 && parallel.size() == 10);
    for (std::size_t i = 0; i < 10; ++i) {
        EXPECT(serial[i].size() == 1 && serial[i][0].shape() == fdeep::tensor_shape(10));
        EXPECT(serial[i][0].to_vector() == parallel[i][0].to_vector());
        EXPECT(serial[i][0].to_vector() == serial[0][0].to_vector());
    }
    float sum = 0;
    for (float v : *serial[0][0].as_vector())
        sum += v;
    EXPECT(std::fabs(sum - 1.0f) < 1e-5f);

    // a non-constant input: predict and predict_class agree, first maximum wins
    fdeep::tensor x(fdeep::tensor_shape(32, 32, 3), 0.0f);
    for (std::size_t y = 0; y < 32; ++y)
        for (std::size_t xx = 0; xx < 32; ++xx)
            for (std::size_t z = 0; z < 3; ++z)
                x.set(fdeep::tensor_pos(y, xx, z), std::sin(0.37f * static_cast<float>(y * 96 + xx * 3 + z)));
    const auto out = model.predict({ x });
    const auto cls = model.predict_class_with_confidence({ x });
    std::size_t best = 0;
    for (std::size_t i = 1; i < 10; ++i)
        if (out[0].get(fdeep::tensor_pos(i)) > out[0].get(fdeep::tensor_pos(best)))
            best = i;
    EXPECT(cls.first == best && cls.second == out[0].get(fdeep::tensor_pos(best)));
    EXPECT(model.predict_class({ x }) == best);
    if (argc > 2)
        EXPECT(static_cast<long>(best) == std::atol(argv[2]));
    EXPECT(model.test_speed() > 0.0);

    // copies share the resident model
    const fdeep::model copy = model;
    EXPECT(copy.predict({ x })[0].to_vector() == out[0].to_vector());

    // predict is const and thread-safe (FAQ.md:103-114): four host threads on one model and on a copy of it, each
    // mixing predict and predict_multi, get what the serial calls above returned
    {
        int bad[4] = { 0, 0, 0, 0 };
        std::vector<std::thread> workers;
        for (int t = 0; t < 4; ++t)
            workers.emplace_back([&, t] {
                const fdeep::model& mine = (t % 2) ? copy : model;
                for (int it = 0; it < 20; ++it) {
                    if (mine.predict({ x })[0].to_vector() != out[0].to_vector())
                        ++bad[t];
                    const auto multi = mine.predict_multi(std::vector<fdeep::tensors>(3 + t, dummy), it % 2 == 0);
                    for (const auto& r : multi)
                        if (r[0].to_vector() != serial[0][0].to_vector())
                            ++bad[t];
                }
            });
        for (auto& w : workers)
            w.join();
        EXPECT(bad[0] + bad[1] + bad[2] + bad[3] == 0);
    }

    // error behaviour (include/fdeep/model.hpp:137-139, 293; tensor_shape.hpp:246-250)
    EXPECT(throws_with([&] { model.predict({ fdeep::tensor(fdeep::tensor_shape(32, 32, 4), 0.0f) }); }, "Invalid inputs shape"));
    EXPECT(throws_with([&] { model.predict({ fdeep::tensor(fdeep::tensor_shape(3072), 0.0f) }); }, "Invalid inputs shape"));
    EXPECT(throws_with([&] { fdeep::load_model("/nonexistent/model.json"); }, "Can not open"));
    EXPECT(throws_with([&] { fdeep::read_model_from_string("{\"image_data_format\": \"channels_first\"}", true, fdeep::dev_null_logger); },
        "only channels_last data format supported"));
    EXPECT(throws_with([&] { model.predict_single_output({ x }); }, "invalid output shape"));

    // byte helpers round-trip
    const std::uint8_t px[6] = { 0, 51, 102, 153, 204, 255 };
    const auto t = fdeep::tensor_from_bytes(px, 1, 2, 3, 0.0f, 1.0f);
    EXPECT(std::fabs(t.get(fdeep::tensor_pos(0, 1, 2)) - 1.0f) < 1e-6f);
    const auto back = fdeep::tensor_to_bytes(t);
    for (int i = 0; i < 6; ++i)
        EXPECT(back[static_cast<std::size_t>(i)] == px[i]);
    EXPECT(fdeep::show_tensor_shape(t.shape()) == "3(1, 2, 3)");
    // show_tensor pads every value to the longest one (include/fdeep/tensor.hpp:1203-1218)
    EXPECT(fdeep::show_tensor(fdeep::tensor(fdeep::tensor_shape(2, 2), std::vector<float> { 1.5f, -12.25f, 0.0f, 3.0f }))
        == "[[[[[  1.5000, -12.2500], [  0.0000,   3.0000]]]]]");
    // dimensions() covers the rank only (include/fdeep/tensor_shape.hpp:153-164)
    EXPECT((fdeep::tensor_shape(7, 5).dimensions() == std::vector<std::size_t> { 7, 5 }));
    EXPECT((fdeep::tensor_pos(1, 2, 3).dimensions() == std::vector<std::size_t> { 1, 2, 3 }));

    // custom layer: a class the device path does not know, created through custom_layer_creators
    // (the reference's FAQ example shape: a layer subclass with apply_impl, registered by class name)
    if (argc > 3) {
        class scale_shift_layer : public fdeep::internal::layer {
        public:
            scale_shift_layer(const std::string& name, const fdeep::float_vec& offset)
                : layer(name)
                , offset_(offset)
            {
            }
            fdeep::tensors apply_impl(const fdeep::tensors& inputs) const override
            {
                fdeep::float_vec v = *inputs.at(0).as_vector();
                for (std::size_t i = 0; i < v.size(); ++i)
                    v[i] = 2.0f * v[i] + offset_[i % offset_.size()];
                return { fdeep::tensor(inputs[0].shape(), std::move(v)) };
            }
            fdeep::float_vec offset_;
        };
        int created = 0;
        const fdeep::internal::layer_creators creators = { { "ScaleShift",
            [&created](const fdeep::internal::get_param_f& get_param, const std::string& layer_json, const std::string& name) {
                ++created;
                if (layer_json.find("\"ScaleShift\"") == std::string::npos)
                    throw std::runtime_error("layer json not passed");
                return std::make_shared<scale_shift_layer>(name, get_param(name, "offset"));
            } } };
        EXPECT(throws_with([&] { fdeep::load_model(argv[3], true, fdeep::dev_null_logger); }, "unknown layer type: ScaleShift"));
        // the file's embedded test (written by the oracle with the same layer semantics) is replayed on load
        const auto custom = fdeep::load_model(argv[3], true, fdeep::dev_null_logger, static_cast<fdeep::float_type>(0.00001), creators);
        EXPECT(created == 1);
        const std::vector<fdeep::tensors> batch(3, custom.generate_dummy_inputs());
        const auto outs = custom.predict_multi(batch, true);
        EXPECT(outs.size() == 3 && outs[0][0].to_vector() == outs[2][0].to_vector());
    }
    std::printf("facade_test ok\n");
    return 0;
}

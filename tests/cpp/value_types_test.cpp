// The value types of the facade, checked against the semantics of the reference's own classes (no GPU work):
// tensor (include/fdeep/tensor.hpp:28-168), tensor_shape (tensor_shape.hpp:100-164), tensor_shape_variable
// (tensor_shape_variable.hpp:87-90), tensor_pos (tensor_pos.hpp:116-147), reshape_tensor_vectors (tensor.hpp:1282-1303).
#include <cstdio>
#include <fdeep/fdeep.hpp>

#define EXPECT(cond)                                                     \
    do {                                                                 \
        if (!(cond)) {                                                   \
            std::fprintf(stderr, "FAILED %s:%d %s\n", __FILE__, __LINE__, #cond); \
            return 1;                                                    \
        }                                                                \
    } while (0)

template <typename F>
static bool throws(F f)
{
    try {
        f();
    } catch (const std::runtime_error&) {
        return true;
    }
    return false;
}

int main()
{
    using namespace fdeep;
    // a 2 x 3 x 4 tensor holding its own flat index
    tensor t(tensor_shape(2, 3, 4), 0.0f);
    for (std::size_t y = 0; y < 2; ++y)
        for (std::size_t x = 0; x < 3; ++x)
            for (std::size_t z = 0; z < 4; ++z)
                t.set(tensor_pos(y, x, z), static_cast<float>((y * 3 + x) * 4 + z));
    // five-index get / set ignore the rank
    EXPECT(t.get(0, 0, 1, 2, 3) == 23.0f);
    t.set(0, 0, 1, 0, 1, -5.0f);
    EXPECT(t.get(tensor_pos(1, 0, 1)) == -5.0f);
    // references into the shared buffer
    t.get_ref_ignore_rank(tensor_pos(0, 0, 1, 0, 1)) = 13.0f;
    const tensor& ct = t;
    EXPECT(ct.get_ref_ignore_rank(tensor_pos(1, 0, 1)) == 13.0f);
    EXPECT(&ct.get_ref_ignore_rank(tensor_pos(1, 0, 1)) == &(*t.as_vector())[13]);
    // padded access: the pad value outside, on every side of every axis
    EXPECT(t.get_padded(7.5f, 0, 0, 1, 2, 3) == 23.0f);
    EXPECT(t.get_padded(7.5f, 0, 0, -1, 0, 0) == 7.5f && t.get_padded(7.5f, 0, 0, 2, 0, 0) == 7.5f);
    EXPECT(t.get_padded(7.5f, 0, 0, 0, -1, 0) == 7.5f && t.get_padded(7.5f, 0, 0, 0, 3, 0) == 7.5f);
    EXPECT(t.get_padded(7.5f, 0, 0, 0, 0, -1) == 7.5f && t.get_padded(7.5f, 0, 0, 0, 0, 4) == 7.5f);
    EXPECT(t.get_padded(7.5f, 1, 0, 0, 0, 0) == 7.5f && t.get_padded(7.5f, 0, -1, 0, 0, 0) == 7.5f);
    // a position of the wrong rank is refused by get / set, not by the _ignore_rank forms
    EXPECT(throws([&] { t.get(tensor_pos(1, 2)); }));
    EXPECT(t.get_ignore_rank(tensor_pos(2, 3)) == 11.0f);
    // rank handling of the tensor follows its shape
    tensor r(tensor_shape(1, 1, 5), 1.0f);
    EXPECT(r.rank() == 3);
    r.shrink_rank();
    EXPECT(r.rank() == 1 && r.shape() == tensor_shape(5));
    r.maximize_rank();
    EXPECT(r.rank() == 5 && r.shape() == tensor_shape(1, 1, 1, 1, 5));
    r.shrink_rank_with_min(2);
    EXPECT(r.rank() == 2 && r.shape() == tensor_shape(1, 5));
    tensor_shape s(1, 1, 4, 1, 1);
    s.shrink_rank_with_min(1);
    EXPECT(s.rank() == 3 && s.minimal_rank() == 3);
    s.shrink_rank_with_min(4);
    EXPECT(s.rank() == 4 && (s.dimensions() == std::vector<std::size_t> { 1, 4, 1, 1 }));
    // unknown extents count as one
    EXPECT(tensor_shape_variable(3, { 1, 1, -1, -1, 3 }).minimal_volume() == 3);
    EXPECT(tensor_shape_variable(2, { 1, 1, 1, 7, 5 }).minimal_volume() == 35);
    // positions from dimension lists
    const tensor_pos p3 = create_tensor_pos_from_dims({ 1, 2, 3 });
    EXPECT(p3.rank() == 3 && p3.y_ == 1 && p3.x_ == 2 && p3.z_ == 3);
    const tensor_pos p5 = create_tensor_pos_from_dims({ 4, 3, 2, 1, 0 });
    EXPECT(p5.rank() == 5 && p5.pos_dim_5_ == 4 && p5.pos_dim_4_ == 3 && p5.y_ == 2 && p5.x_ == 1 && p5.z_ == 0);
    EXPECT(create_tensor_pos_from_dims({ 9 }).z_ == 9 && create_tensor_pos_from_dims({ 8, 9 }).x_ == 8);
    EXPECT((create_tensor_pos_from_dims({ 6, 7, 8, 9 }).dimensions() == std::vector<std::size_t> { 6, 7, 8, 9 }));
    EXPECT(throws([] { create_tensor_pos_from_dims({}); }));
    EXPECT(throws([] { create_tensor_pos_from_dims({ 1, 2, 3, 4, 5, 6 }); }));
    // reshape_tensor_vectors: 24 values as 2 vectors of 3 tensors of shape (1, 2, 2), order kept
    tensors_vec in;
    in.push_back({ tensor(tensor_shape(6), float_vec { 0, 1, 2, 3, 4, 5 }), tensor(tensor_shape(2, 3), float_vec { 6, 7, 8, 9, 10, 11 }) });
    in.push_back({ tensor(tensor_shape(12), float_vec { 12, 13, 14, 15, 16, 17, 18, 19, 20, 21, 22, 23 }) });
    const tensors_vec out = reshape_tensor_vectors(2, 3, 2, 1, 2, in);
    EXPECT(out.size() == 2 && out[0].size() == 3 && out[1].size() == 3);
    float next = 0.0f;
    for (const auto& ts : out)
        for (const auto& one : ts) {
            EXPECT(one.shape() == tensor_shape(1, 2, 2));
            for (float v : *one.as_vector())
                EXPECT(v == next++);
        }
    EXPECT(throws([&] { reshape_tensor_vectors(2, 3, 2, 1, 3, in); }));
    // the non-const buffer handle can be swapped for another buffer of the same size
    tensor sw(tensor_shape(3), 0.0f);
    sw.as_vector() = std::make_shared<float_vec>(float_vec { 1, 2, 3 });
    EXPECT(sw.get(tensor_pos(2)) == 3.0f);
    std::printf("value_types_test ok\n");
    return 0;
}

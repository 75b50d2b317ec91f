// Decode attention for the common head shape (key_dim = value_dim = 64, at most 256 cached
// positions): one query row per (sequence, head) against the token-major key / value cache.
//
// The kernel is one memory round trip: every lane issues all of its key AND value loads
// (16 bytes each, sixteen lanes per cached row so a wave touches four whole rows per load)
// before anything is used; the values do not depend on the softmax, so they travel while the
// scores are reduced.  Scores stay in registers; max / sum / output reductions use wave
// shuffles and ONE small LDS exchange between the four waves.  Softmax weights equal the
// reference's exp(x - m - log(sum)) (include/fdeep/tensor.hpp:1165-1192) up to rounding; the
// scale multiplies the scores after the dot product (layers/multi_head_attention_layer.hpp:91-93).
#include <cfloat>
#include <cmath>

#include "common.hpp"
#include "global_ptr.hpp"
#include "skinny.hpp"

namespace fdx {

typedef float f32x4 __attribute__((ext_vector_type(4)));

#include "decode_attn_body.hpp"

__global__ __launch_bounds__(256) void mha_decode_fast_kernel(const float* __restrict__ q, int64_t ldq,
    const float* __restrict__ kc, const float* __restrict__ vc, float* __restrict__ out, int heads,
    const int* __restrict__ len_dev, int max_len, float scale)
{
    __shared__ MhaDecodeShared sh;
    mha_decode_fast_body<false>(q, ldq, kc, vc, out, heads, len_dev, max_len, scale, blockIdx.x, threadIdx.x, true, sh);
}

// true if the fast kernel covers this shape; launches it
bool mha_decode_fast_launch(const float* q, int64_t ldq, const float* kc, const float* vc, float* out, int batch, int heads,
    int dk, int dv, const int* len_dev, int max_len, hipStream_t s)
{
    if (dk != 64 || dv != 64 || max_len > 256 || ldq % 4 != 0)
        return false;
    const float scale = (float)(1.0 / std::sqrt((double)dk));
    hipLaunchKernelGGL(mha_decode_fast_kernel, dim3(batch * heads), dim3(256), 0, s, q, ldq, kc, vc, out, heads, len_dev, max_len, scale);
    return true;
}

} // namespace fdx

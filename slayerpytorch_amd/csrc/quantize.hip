// Weight quantisation of the Loihi layers: round(w / step) * step (src/quantizeParams.py:3-31), one launch
// instead of the three element-wise launches of the tensor expression.  The layers quantise their weights
// in every forward pass, and the tensors are small: the launches, not the arithmetic, are what it costs.
#include "common.h"

namespace slayer {

// What torch makes of `tensor / number` on the GPU is a product with the reciprocal of the number, taken in double
// precision and rounded to fp32; then to the nearest integer with ties to even (torch.round), then * step in fp32.
__global__ __launch_bounds__(256) void quantize_kernel(float *__restrict__ out, const float *__restrict__ in, int64_t n,
                                                       float inverse, float step)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) out[i] = rintf(in[i] * inverse) * step;
}

}  // namespace slayer

extern "C" int slayer_quantize_f32(float *out, const float *in, int64_t n, double step, void *stream)
{
    using namespace slayer;
    if (n < 0) return SLAYER_EINVAL;
    if (n == 0) return SLAYER_OK;
    if (!out || !in) return SLAYER_EINVAL;
    const int64_t blocks = ceil_div(n, 256);
    if (blocks >= (1LL << 24)) return SLAYER_EUNSUPPORTED;
    hipLaunchKernelGGL(quantize_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       out, in, n, static_cast<float>(1.0 / step), static_cast<float>(step));
    return launch_status();
}

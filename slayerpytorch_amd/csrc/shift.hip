// Time shift of neuron rows: out[n][t] = in[n][t - k_n], zero outside [0, T).
//
// HBM-bound gather (8 B per neuron-timestep: one read, one write).  A work-group owns a
// block of consecutive rows, i.e. one contiguous piece of the tensor; every lane writes one
// 16-byte vector of the output, so stores are fully coalesced, and reads the (generally
// unaligned) source samples from the same row.  The delay of a row is either one value for
// the whole tensor or an entry of a per-neuron table shared by all batch items; one launch
// covers every batch item.
#include "common.h"

namespace slayer {

enum ShiftMode { kShiftValue = 0, kShiftDeviceScalar = 1, kShiftTable = 2 };

// VEC = samples written per lane (4 when rows are 16-byte aligned multiples of 4 samples).
template <int VEC>
__global__ __launch_bounds__(256) void shift_kernel(float *__restrict__ out,
                                                    const float *__restrict__ in,
                                                    const float *__restrict__ lut, int mode,
                                                    float delayValue, float sign, int64_t rows,
                                                    uint32_t nPerBatch, int T, int rowsPerBlock,
                                                    float Ts)
{
    const int perRow = T / VEC;  // vectors per row
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * rowsPerBlock;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(rowsPerBlock), rows - row0));
    const int items = nRows * perRow;
    const float invPerRow = 1.0f / static_cast<float>(perRow);
    const uint32_t m0 = (mode == kShiftTable) ? static_cast<uint32_t>(row0 % nPerBatch) : 0u;

    int uniformSteps = 0;
    if (mode == kShiftValue) uniformSteps = delay_steps(delayValue * sign, Ts);
    if (mode == kShiftDeviceScalar) uniformSteps = delay_steps(lut[0] * sign, Ts);

    for (int i = threadIdx.x; i < items; i += blockDim.x) {
        int r = 0, q = i;
        if (nRows > 1) {
            // i / perRow for i < 2^24: float estimate plus one correction step
            r = static_cast<int>(static_cast<float>(i) * invPerRow);
            q = i - r * perRow;
            if (q < 0) { --r; q += perRow; }
            else if (q >= perRow) { ++r; q -= perRow; }
        }
        int k = uniformSteps;
        if (mode == kShiftTable) {
            uint32_t m = (m0 + static_cast<uint32_t>(r)) % nPerBatch;
            k = delay_steps(lut[m] * sign, Ts);
        }
        const int64_t base = (row0 + r) * static_cast<int64_t>(T);
        const float *src = in + base;
        const int t = q * VEC;
        // source sample index of the first output sample; 64-bit so that t - k cannot wrap
        const int64_t s0 = static_cast<int64_t>(t) - k;
        if (VEC == 4) {
            float4 v;
            if ((k & 3) == 0 && s0 >= 0 && s0 + 3 < T) {
                v = *reinterpret_cast<const float4 *>(src + s0);
            } else {
                v.x = (s0 >= 0 && s0 < T) ? src[s0] : 0.0f;
                v.y = (s0 + 1 >= 0 && s0 + 1 < T) ? src[s0 + 1] : 0.0f;
                v.z = (s0 + 2 >= 0 && s0 + 2 < T) ? src[s0 + 2] : 0.0f;
                v.w = (s0 + 3 >= 0 && s0 + 3 < T) ? src[s0 + 3] : 0.0f;
            }
            *reinterpret_cast<float4 *>(out + base + t) = v;
        } else {
            out[base + t] = (s0 >= 0 && s0 < T) ? src[s0] : 0.0f;
        }
    }
}

static int launch_shift(float *out, const float *in, const float *lut, int mode, float delayValue,
                        float sign, int64_t rows, int64_t nPerBatch, int64_t T, float Ts,
                        hipStream_t stream)
{
    if (rows < 0 || T < 0 || nPerBatch < 0) return SLAYER_EINVAL;
    if (rows == 0 || T == 0) return SLAYER_OK;
    if (!out || !in) return SLAYER_EINVAL;
    if (mode != kShiftValue && !lut) return SLAYER_EINVAL;
    if (T >= (1LL << 30) || nPerBatch >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    if (mode == kShiftTable && nPerBatch == 0) return SLAYER_EINVAL;

    const bool vec4 = (T % 4 == 0) && aligned16(out) && aligned16(in);
    const int vec = vec4 ? 4 : 1;
    const int64_t perRow = T / vec;
    // about 2048 vectors (8 per lane) per work-group, whole rows only, and the in-block
    // item index must stay below 2^24 for the float division in the kernel
    int64_t rowsPerBlock = perRow >= 2048 ? 1 : (2048 / perRow);
    if (rowsPerBlock > rows) rowsPerBlock = rows;
    const int64_t blocks = ceil_div(rows, rowsPerBlock);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;

    dim3 grid(static_cast<unsigned>(blocks)), block(256);
    if (vec4)
        hipLaunchKernelGGL(shift_kernel<4>, grid, block, 0, stream, out, in, lut, mode, delayValue,
                           sign, rows, static_cast<uint32_t>(nPerBatch), static_cast<int>(T),
                           static_cast<int>(rowsPerBlock), Ts);
    else
        hipLaunchKernelGGL(shift_kernel<1>, grid, block, 0, stream, out, in, lut, mode, delayValue,
                           sign, rows, static_cast<uint32_t>(nPerBatch), static_cast<int>(T),
                           static_cast<int>(rowsPerBlock), Ts);
    return launch_status();
}

}  // namespace slayer

extern "C" int slayer_shift_f32(float *out, const float *in, float delay, int64_t nNeurons,
                                int64_t T, float Ts, void *stream)
{
    return slayer::launch_shift(out, in, nullptr, slayer::kShiftValue, delay, 1.0f, nNeurons, 1, T,
                                Ts, static_cast<hipStream_t>(stream));
}

extern "C" int slayer_shift_lut_f32(float *out, const float *in, const float *lut, int64_t lutSize,
                                    int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts,
                                    float sign, void *stream)
{
    if (nBatch < 0 || nPerBatch < 0 || lutSize < 0) return SLAYER_EINVAL;
    if (!(sign == 1.0f || sign == -1.0f)) return SLAYER_EINVAL;
    const int64_t rows = nBatch * nPerBatch;
    if (lutSize == 1)
        return slayer::launch_shift(out, in, lut, slayer::kShiftDeviceScalar, 0.0f, sign, rows, 1, T,
                                    Ts, static_cast<hipStream_t>(stream));
    if (rows != 0 && T != 0 && lutSize != nPerBatch) return SLAYER_EINVAL;
    return slayer::launch_shift(out, in, lut, slayer::kShiftTable, 0.0f, sign, rows, nPerBatch, T,
                                Ts, static_cast<hipStream_t>(stream));
}

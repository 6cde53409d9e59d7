// Time shift of neuron rows: out[n][t] = in[n][t - k_n], zero outside [0, T).
//
// HBM-bound gather (8 B per neuron-timestep: one read, one write), built like the fastest copy
// this GPU runs: one 16-byte vector per lane, one pass per work-group, streaming cache policy.
// A work-group owns a few whole rows (or a 256-vector slice of a long row); a lane writes one
// aligned output vector and assembles it from the two aligned input vectors that straddle its
// shifted position, so both directions stay fully coalesced whatever the shift is.  The delay
// of a row is either one value for the whole tensor or an entry of a per-neuron table shared
// by all batch items; one launch covers every batch item.
#include "common.h"

namespace slayer {

enum ShiftMode { kShiftValue = 0, kShiftDeviceScalar = 1, kShiftTable = 2 };

// Delay, in whole samples, of row (row0 + r); r < 256.  The table index is the row's position
// within its batch item: the 64-bit remainder is taken once per work-group (row0 is uniform),
// the per-lane part is 32 bit.
__device__ __forceinline__ int row_steps(int mode, const float *__restrict__ lut, float delayValue,
                                         float sign, float Ts, int64_t row0, int r, uint32_t nPerBatch)
{
    if (mode == kShiftValue) return delay_steps(delayValue * sign, Ts);
    if (mode == kShiftDeviceScalar) return delay_steps(lut[0] * sign, Ts);
    const uint32_t m0 = static_cast<uint32_t>(row0 % static_cast<int64_t>(nPerBatch));
    const uint32_t m = static_cast<uint32_t>((static_cast<uint64_t>(m0) + static_cast<uint32_t>(r)) % nPerBatch);
    return delay_steps(lut[m] * sign, Ts);
}

// Rows are whole 16-byte vectors (T % 4 == 0, 16-byte aligned tensors) and the tensor has fewer
// than 2^32 of them: lane g of the grid owns output vector g of the flattened tensor.
template <int LOADPOLICY>
__global__ __launch_bounds__(256) void shift_vec_kernel(float *__restrict__ out,
                                                        const float *__restrict__ in,
                                                        const float *__restrict__ lut, int mode,
                                                        float delayValue, float sign, uint32_t quads,
                                                        uint32_t nPerBatch, int T, FastDiv byRow,
                                                        float Ts)
{
    const int perRow = T >> 2;
    const uint32_t g0 = blockIdx.x * 256u;      // first vector of this work-group
    const uint32_t g = g0 + threadIdx.x;
    const bool active = g < quads;
    const uint32_t rowBase = fastdiv(g0, byRow);  // wave-uniform: addressing is relative to this row
    const uint32_t row = fastdiv(active ? g : g0, byRow);
    const int q = static_cast<int>((active ? g : g0) - row * static_cast<uint32_t>(perRow));
    const int r = static_cast<int>(row - rowBase);

    const BufferRsrc bufIn = make_buffer(in + static_cast<int64_t>(rowBase) * T);
    const BufferRsrc bufOut = make_buffer(out + static_cast<int64_t>(rowBase) * T);
    int k = row_steps(mode, lut, delayValue, sign, Ts, rowBase, r, nPerBatch);
    k = max(-T, min(T, k));             // shifts beyond the row length all give an empty row
    const int s0 = (q << 2) - k;        // source sample of the first output sample
    const int qa = s0 >> 2;             // aligned source vector holding it (floor division)
    const int sh = s0 & 3;
    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    float4 a = zero, b = zero;
    if (active && qa >= 0 && qa < perRow) a = buffer_load4<LOADPOLICY>(bufIn, (r * T + (qa << 2)) * 4, 0);
    if (active && sh != 0 && qa + 1 >= 0 && qa + 1 < perRow)
        b = buffer_load4<LOADPOLICY>(bufIn, (r * T + (qa << 2) + 4) * 4, 0);
    float4 y = a;
    if (sh == 1) y = make_float4(a.y, a.z, a.w, b.x);
    if (sh == 2) y = make_float4(a.z, a.w, b.x, b.y);
    if (sh == 3) y = make_float4(a.w, b.x, b.y, b.z);
    if (active) buffer_store4(bufOut, (r * T + (q << 2)) * 4, 0, y);
}

// Rows that are not whole 16-byte vectors (T % 4 != 0) in a tensor that is (16-byte aligned,
// rows * T % 4 == 0, T >= 4, fewer than 2^31 samples): lane g still owns the aligned output
// vector g of the flattened tensor, which now may hold the end of one row and the start of the
// next.  Each of the (at most two) row parts is assembled like in the kernel above, from the two
// aligned input vectors that straddle its shifted position; only the lanes whose vector spans
// two rows, one in T/4, take the second turn.
__global__ __launch_bounds__(256) void shift_flat_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                         const float *__restrict__ lut, int mode, float delayValue,
                                                         float sign, uint32_t quads, uint32_t nPerBatch, int T,
                                                         FastDiv byT, FastDiv byBatch, float Ts)
{
    const uint32_t g = blockIdx.x * 256u + threadIdx.x;
    if (g >= quads) return;
    const float4 *vin = reinterpret_cast<const float4 *>(in);
    const uint32_t e0 = g << 2;                          // first sample of the vector, flat
    const uint32_t rowA = fastdiv(e0, byT);
    const int tA = static_cast<int>(e0 - rowA * static_cast<uint32_t>(T));
    const int nA = min(4, T - tA);                       // samples of the vector that belong to rowA

    float y[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    // samples j0 .. j0+count-1 of the vector are the samples tStart .. of `row`
    auto part = [&](uint32_t row, int tStart, int j0, int count) {
        int k;
        if (mode == kShiftValue) k = delay_steps(delayValue * sign, Ts);
        else if (mode == kShiftDeviceScalar) k = delay_steps(lut[0] * sign, Ts);
        else k = delay_steps(lut[row - fastdiv(row, byBatch) * nPerBatch] * sign, Ts);
        k = max(-T, min(T, k));
        // the vector's sample j comes from flat position q + j
        const int q = static_cast<int>(row) * T + tStart - k - j0;
        const int va = q >> 2, sh = q & 3;               // floor division
        const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        float4 a = zero, b = zero;
        if (va >= 0 && va < static_cast<int>(quads)) a = vin[va];
        if (sh != 0 && va + 1 >= 0 && va + 1 < static_cast<int>(quads)) b = vin[va + 1];
        float c[4] = {a.x, a.y, a.z, a.w};
        if (sh == 1) { c[0] = a.y; c[1] = a.z; c[2] = a.w; c[3] = b.x; }
        if (sh == 2) { c[0] = a.z; c[1] = a.w; c[2] = b.x; c[3] = b.y; }
        if (sh == 3) { c[0] = a.w; c[1] = b.x; c[2] = b.y; c[3] = b.z; }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int src = tStart + (j - j0) - k;       // source time within the row
            if (j >= j0 && j < j0 + count && src >= 0 && src < T) y[j] = c[j];
        }
    };
    part(rowA, tA, 0, nA);
    if (nA < 4) part(rowA + 1, 0, nA, 4 - nA);
    typedef float vec4f __attribute__((ext_vector_type(4)));
    const vec4f o = {y[0], y[1], y[2], y[3]};
    __builtin_nontemporal_store(o, reinterpret_cast<vec4f *>(out) + g);
}

// Any T, any alignment: one sample per lane, lanes along time (coalesced 256-byte runs).
__global__ __launch_bounds__(256) void shift_scalar_kernel(float *__restrict__ out,
                                                           const float *__restrict__ in,
                                                           const float *__restrict__ lut, int mode,
                                                           float delayValue, float sign, int64_t rows,
                                                           uint32_t nPerBatch, int T, int rowsPerBlock,
                                                           float Ts)
{
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * rowsPerBlock;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(rowsPerBlock), rows - row0));
    int r = 0, t = blockIdx.y * 256 + threadIdx.x;
    if (rowsPerBlock > 1) divmod_small(threadIdx.x, T, 1.0f / static_cast<float>(T), r, t);
    if (r >= nRows || t >= T) return;
    int k = row_steps(mode, lut, delayValue, sign, Ts, row0, r, nPerBatch);
    k = max(-T, min(T, k));
    const int src = t - k;
    const int64_t base = (row0 + r) * static_cast<int64_t>(T);
    out[base + t] = (src >= 0 && src < T) ? in[base + src] : 0.0f;
}

static int launch_shift(float *out, const float *in, const float *lut, int mode, float delayValue,
                        float sign, int64_t rows, int64_t nPerBatch, int64_t T, float Ts,
                        hipStream_t stream)
{
    if (rows < 0 || T < 0 || nPerBatch < 0) return SLAYER_EINVAL;
    if (rows == 0 || T == 0) return SLAYER_OK;
    if (!out || !in) return SLAYER_EINVAL;
    if (mode != kShiftValue && !lut) return SLAYER_EINVAL;
    if (T >= (1LL << 28) || nPerBatch >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    if (mode == kShiftTable && nPerBatch == 0) return SLAYER_EINVAL;

    const bool vec = (T % 4 == 0) && aligned16(out) && aligned16(in) && rows * (T / 4) < (1LL << 32);
    if (vec) {
        const int64_t quads = rows * (T / 4);
        const int64_t blocks = ceil_div(quads, 256);
        // an aligned shift (whole vectors) reads every input vector exactly once: stream it;
        // otherwise neighbouring lanes share input vectors and the loads should stay cached
        hipLaunchKernelGGL(shift_vec_kernel<0>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream, out,
                           in, lut, mode, delayValue, sign, static_cast<uint32_t>(quads),
                           static_cast<uint32_t>(nPerBatch), static_cast<int>(T),
                           make_fastdiv(static_cast<uint32_t>(T / 4)), Ts);
        return launch_status();
    }
    if (T % 4 != 0 && T >= 4 && aligned16(out) && aligned16(in) && (rows * T) % 4 == 0 && rows * T < (1LL << 31)) {
        const int64_t quads = rows * T / 4;
        hipLaunchKernelGGL(shift_flat_kernel, dim3(static_cast<unsigned>(ceil_div(quads, 256))), dim3(256), 0, stream,
                           out, in, lut, mode, delayValue, sign, static_cast<uint32_t>(quads),
                           static_cast<uint32_t>(nPerBatch), static_cast<int>(T), make_fastdiv(static_cast<uint32_t>(T)),
                           make_fastdiv(static_cast<uint32_t>(nPerBatch > 0 ? nPerBatch : 1)), Ts);
        return launch_status();
    }
    const int64_t rowsPerBlock = T >= 256 ? 1 : 256 / T;
    const int64_t rowBlocks = ceil_div(rows, rowsPerBlock);
    const int64_t colBlocks = ceil_div(T, 256);
    if (rowBlocks >= (1LL << 31) || colBlocks > 65535) return SLAYER_EUNSUPPORTED;
    dim3 grid(static_cast<unsigned>(rowBlocks), static_cast<unsigned>(rowsPerBlock > 1 ? 1 : colBlocks));
    hipLaunchKernelGGL(shift_scalar_kernel, grid, dim3(256), 0, stream, out, in, lut, mode, delayValue, sign,
                       rows, static_cast<uint32_t>(nPerBatch), static_cast<int>(T),
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

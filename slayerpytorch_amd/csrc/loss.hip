// Spike-train loss of the output layer in two launches: the error signal
// error = psp(out - desired) [+ addend] and loss = 1/2 * sum(error^2) * Ts, which the reference
// evaluates as a chain of tensor expressions (src/spikeLoss.py:56-58 and :100-104).  The output layer
// is tiny (classes x batch rows), so the cost of that chain is its launches, not its bytes.
#include "common.h"

namespace slayer {

// One work-group per row.  The row of differences sits in LDS behind F-1 zeros, so every output is
// the full tap chain acc = fma(d[t-k], srm[k], acc), k = 0 .. F-1, then * Ts - the arithmetic of the
// temporal convolution kernels, bit for bit (taps that reach before the row multiply a zero).
__global__ __launch_bounds__(256) void spike_loss_rows_kernel(float *__restrict__ error, float *__restrict__ partial,
                                                              const float *__restrict__ out,
                                                              const float *__restrict__ desired,
                                                              const float *__restrict__ addend,
                                                              const float *__restrict__ srm, int T, int F, float Ts)
{
    extern __shared__ float lds[];
    float *filt = lds;          // [F]
    float *diff = lds + F;      // [F - 1 zeros][T]
    __shared__ float wsum[4];
    const int64_t base = static_cast<int64_t>(blockIdx.x) * T;
    for (int k = threadIdx.x; k < F; k += 256) filt[k] = srm[k];
    for (int i = threadIdx.x; i < F - 1 + T; i += 256) {
        const int t = i - (F - 1);
        diff[i] = t >= 0 ? out[base + t] - desired[base + t] : 0.0f;
    }
    __syncthreads();
    float sq = 0.0f;
    for (int t = threadIdx.x; t < T; t += 256) {
        const float *d = diff + (F - 1) + t;
        float acc = 0.0f;
        for (int k = 0; k < F; ++k) acc = fmaf(d[-k], filt[k], acc);
        float e = acc * Ts;
        if (addend) e += addend[base + t];
        error[base + t] = e;
        sq = fmaf(e, e, sq);
    }
    // fixed-shape reduction: lanes of a wavefront, then the four wavefronts in order
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) sq += __shfl_down(sq, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0) wsum[threadIdx.x / kWave] = sq;
    __syncthreads();
    if (threadIdx.x == 0) partial[blockIdx.x] = ((wsum[0] + wsum[1]) + wsum[2]) + wsum[3];
}

// loss = scale * sum of the row sums: lane l adds rows l, l+256, ... in order, then a fixed tree.
__global__ __launch_bounds__(256) void spike_loss_sum_kernel(float *__restrict__ loss, const float *__restrict__ partial,
                                                             int64_t rows, float scale)
{
    __shared__ float wsum[4];
    float acc = 0.0f;
    for (int64_t r = threadIdx.x; r < rows; r += 256) acc += partial[r];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) acc += __shfl_down(acc, off, kWave);
    if ((threadIdx.x & (kWave - 1)) == 0) wsum[threadIdx.x / kWave] = acc;
    __syncthreads();
    if (threadIdx.x == 0) loss[0] = (((wsum[0] + wsum[1]) + wsum[2]) + wsum[3]) * scale;
}

}  // namespace slayer

extern "C" int64_t slayer_spike_loss_workspace_bytes(int64_t rows)
{
    return rows > 0 ? rows * static_cast<int64_t>(sizeof(float)) : 0;
}

extern "C" int slayer_spike_loss_f32(float *loss, float *error, const float *out, const float *desired,
                                     const float *addend, const float *srm, float *workspace, int64_t rows,
                                     int64_t T, int64_t F, float Ts, void *stream)
{
    using namespace slayer;
    if (rows < 0 || T < 0 || F < 0) return SLAYER_EINVAL;
    if (!loss) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t live = (rows > 0 && T > 0) ? rows : 0;
    if (live > 0) {
        if (!error || !out || !desired || !workspace || (F > 0 && !srm)) return SLAYER_EINVAL;
        // a row and the filter must fit the LDS of one work-group
        const int64_t ldsBytes = (2 * F + T) * static_cast<int64_t>(sizeof(float));
        if (ldsBytes > 60 * 1024 || live >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
        hipLaunchKernelGGL(spike_loss_rows_kernel, dim3(static_cast<unsigned>(live)), dim3(256),
                           static_cast<size_t>(ldsBytes), st, error, workspace, out, desired, addend, srm,
                           static_cast<int>(T), static_cast<int>(F), Ts);
        const int status = launch_status();
        if (status != SLAYER_OK) return status;
    }
    hipLaunchKernelGGL(spike_loss_sum_kernel, dim3(1), dim3(256), 0, st, loss, workspace, live, 0.5f * Ts);
    return launch_status();
}

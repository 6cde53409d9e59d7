// Gradient of a time shift with respect to its per-neuron delay table:
//
//   gradDelay[m] = Ts * sum_{b,t} gradOut[b][m][t] * d[b][m][t],
//   d[b][m][t]   = out[b][m][t] * (-1/Ts) + out[b][m][t-1] * (1/Ts)        (out[.][.][-1] = 0)
//
// i.e. the 2-tap causal difference of the shifted signal, weighted by the incoming gradient and
// reduced over batch and time.  HBM-bound (8 B per neuron-timestep: both tensors read once).
// Pass 1: one wavefront per neuron row reduces its T products (lanes along time, coalesced) to
// one partial sum in the caller's workspace.  Pass 2: one lane per table entry adds the
// nBatch partials in batch order and scales by Ts.  The summation order is fixed, so results
// are reproducible from run to run.
#include "common.h"

#include <atomic>

namespace slayer {

// VEC: rows are whole 16-byte vectors (T % 4 == 0, 16-byte aligned tensors): a lane takes four
// consecutive samples per trip and gets the sample before them from the lane to its left.
template <bool VEC>
__global__ __launch_bounds__(256) void delay_grad_rows_kernel(float *__restrict__ partial,
                                                              const float *__restrict__ out,
                                                              const float *__restrict__ gradOut,
                                                              int64_t rows, int64_t T, float f0, float f1)
{
    typedef float vec4f __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t wavesPerGrid = static_cast<int64_t>(gridDim.x) * (blockDim.x / kWave);
    for (int64_t row = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
         row < rows; row += wavesPerGrid) {
        const float *y = out + row * T;
        const float *g = gradOut + row * T;
        float acc = 0.0f;
        if (VEC) {
            const int64_t quads = T >> 2;
            for (int64_t q0 = 0; q0 < quads; q0 += kWave) {
                const int64_t q = q0 + lane;
                vec4f yv = {0.0f, 0.0f, 0.0f, 0.0f}, gv = {0.0f, 0.0f, 0.0f, 0.0f};
                if (q < quads) {
                    yv = __builtin_nontemporal_load(reinterpret_cast<const vec4f *>(y) + q);
                    gv = __builtin_nontemporal_load(reinterpret_cast<const vec4f *>(g) + q);
                }
                float before = __shfl_up(yv.w, 1, kWave);   // y[4q - 1] from the lane to the left
                if (lane == 0) before = (q0 > 0) ? y[4 * q0 - 1] : 0.0f;
                const bool first = q == 0;                  // y[-1] does not exist: one-tap difference
                float d0 = yv.x * f0;
                if (!first) d0 = __builtin_fmaf(before, f1, d0);
                const float d1 = __builtin_fmaf(yv.x, f1, yv.y * f0);
                const float d2 = __builtin_fmaf(yv.y, f1, yv.z * f0);
                const float d3 = __builtin_fmaf(yv.z, f1, yv.w * f0);
                acc = __builtin_fmaf(gv.x, d0, acc);
                acc = __builtin_fmaf(gv.y, d1, acc);
                acc = __builtin_fmaf(gv.z, d2, acc);
                acc = __builtin_fmaf(gv.w, d3, acc);
            }
        } else {
            for (int64_t t = lane; t < T; t += kWave) {
                float d = y[t] * f0;
                if (t > 0) d = __builtin_fmaf(y[t - 1], f1, d);
                acc = __builtin_fmaf(g[t], d, acc);
            }
        }
#pragma unroll
        for (int off = kWave / 2; off > 0; off >>= 1) acc += __shfl_down(acc, off, kWave);
        if (lane == 0) partial[row] = acc;
    }
}

// Pass 2, few batch items: one lane per table entry adds the nBatch partials in batch order
// (neighbouring lanes read neighbouring entries).
__global__ __launch_bounds__(256) void delay_grad_batch_kernel(float *__restrict__ gradDelay,
                                                               const float *__restrict__ partial,
                                                               int64_t nBatch, int64_t nPerBatch, float Ts)
{
    const int64_t m = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (m >= nPerBatch) return;
    float acc = 0.0f;
    for (int64_t b = 0; b < nBatch; ++b) acc += partial[b * nPerBatch + m];
    gradDelay[m] = acc * Ts;
}

// Pass 2, many batch items: one wavefront per table entry; lane l adds the partials of batch
// items l, l+64, .. in order, then the 64 lane sums are combined in a fixed tree.
__global__ __launch_bounds__(256) void delay_grad_batch_wave_kernel(float *__restrict__ gradDelay,
                                                                    const float *__restrict__ partial,
                                                                    int64_t nBatch, int64_t nPerBatch, float Ts)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t m = static_cast<int64_t>(blockIdx.x) * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (m >= nPerBatch) return;
    float acc = 0.0f;
    for (int64_t b = lane; b < nBatch; b += kWave) acc += partial[b * nPerBatch + m];
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) acc += __shfl_down(acc, off, kWave);
    if (lane == 0) gradDelay[m] = acc * Ts;
}

}  // namespace slayer

extern "C" int64_t slayer_delay_grad_workspace_bytes(int64_t nBatch, int64_t nPerBatch, int64_t T)
{
    (void)T;
    if (nBatch <= 0 || nPerBatch <= 0) return 0;
    return nBatch * nPerBatch * static_cast<int64_t>(sizeof(float));
}

namespace slayer {

// Partial sums of slayer_delay_grad_static_f32: one float per neuron row.  Every GPU the library runs on
// holds its own copy of this array at its own address until the process ends.
constexpr int64_t kStaticRows = 262144;  // 1 MiB
static __device__ __align__(256) float scratch[kStaticRows];

// The array's address on each device, looked up once per device; host code uses these pointers, never
// the array's name (which is only a handle for the lookup on the host side).
constexpr int kMaxDevices = 64;
static std::atomic<float *> g_scratch_ptr[kMaxDevices];

static int scratch_of_current_device(float **ptr)
{
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return note_hip_error(err);
    if (device < 0 || device >= kMaxDevices) return SLAYER_EUNSUPPORTED;
    float *p = g_scratch_ptr[device].load(std::memory_order_acquire);
    if (!p) {
        void *sym = nullptr;
        err = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return note_hip_error(err);
        if (!sym) return SLAYER_ELAUNCH;
        p = static_cast<float *>(sym);
        g_scratch_ptr[device].store(p, std::memory_order_release);  // (two racing threads store the same address)
    }
    *ptr = p;
    return SLAYER_OK;
}

static int launch_delay_grad(float *gradDelay, const float *out, const float *gradOut, float *workspace, int64_t nBatch,
                             int64_t nPerBatch, int64_t T, float Ts, void *stream);

}  // namespace slayer

extern "C" int slayer_delay_grad_f32(float *gradDelay, const float *out, const float *gradOut,
                                     float *workspace, int64_t nBatch, int64_t nPerBatch, int64_t T,
                                     float Ts, void *stream)
{
    return slayer::launch_delay_grad(gradDelay, out, gradOut, workspace, nBatch, nPerBatch, T, Ts, stream);
}

extern "C" int64_t slayer_delay_grad_static_max_rows(void) { return slayer::kStaticRows; }

extern "C" int slayer_delay_grad_static_f32(float *gradDelay, const float *out, const float *gradOut, int64_t nBatch,
                                            int64_t nPerBatch, int64_t T, float Ts, void *stream)
{
    using namespace slayer;
    if (nBatch < 0 || nPerBatch < 0 || T < 0) return SLAYER_EINVAL;
    // (checked before the product is formed, so that it cannot overflow)
    if (nBatch > kStaticRows || nPerBatch > kStaticRows || nBatch * nPerBatch > kStaticRows) return SLAYER_EUNSUPPORTED;
    float *partial = nullptr;
    const int status = scratch_of_current_device(&partial);
    if (status != SLAYER_OK) return status;
    // every partial sum that pass 2 reads has been written by pass 1 of the same call: nothing to clear
    return launch_delay_grad(gradDelay, out, gradOut, partial, nBatch, nPerBatch, T, Ts, stream);
}

static int slayer::launch_delay_grad(float *gradDelay, const float *out, const float *gradOut, float *workspace,
                                     int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts, void *stream)
{
    if (nBatch < 0 || nPerBatch < 0 || T < 0) return SLAYER_EINVAL;
    if (nPerBatch == 0) return SLAYER_OK;
    if (!gradDelay) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int64_t rows = nBatch * nPerBatch;
    const int64_t outBlocks = ceil_div(nPerBatch, 256);
    if (outBlocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    if (rows > 0 && T > 0) {
        if (!out || !gradOut || !workspace) return SLAYER_EINVAL;
        int64_t blocks = ceil_div(rows, 4);  // four wavefronts (rows) per work-group
        if (blocks > 262144) blocks = 262144;
        if ((T % 4 == 0) && aligned16(out) && aligned16(gradOut))
            hipLaunchKernelGGL(delay_grad_rows_kernel<true>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                               workspace, out, gradOut, rows, T, -1.0f / Ts, 1.0f / Ts);
        else
            hipLaunchKernelGGL(delay_grad_rows_kernel<false>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                               workspace, out, gradOut, rows, T, -1.0f / Ts, 1.0f / Ts);
        int status = launch_status();
        if (status != SLAYER_OK) return status;
    }
    // with no samples to reduce (nBatch == 0 or T == 0) the loop below is empty and yields zeros
    const int64_t batches = (rows > 0 && T > 0) ? nBatch : 0;
    const int64_t waveBlocks = ceil_div(nPerBatch, 4);
    if (batches >= 32 && waveBlocks < (1LL << 31))
        hipLaunchKernelGGL(delay_grad_batch_wave_kernel, dim3(static_cast<unsigned>(waveBlocks)), dim3(256), 0, st,
                           gradDelay, workspace, batches, nPerBatch, Ts);
    else
        hipLaunchKernelGGL(delay_grad_batch_kernel, dim3(static_cast<unsigned>(outBlocks)), dim3(256), 0, st,
                           gradDelay, workspace, batches, nPerBatch, Ts);
    return launch_status();
}

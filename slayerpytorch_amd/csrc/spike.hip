// SRM spike generation: threshold crossing with refractory feedback, sequential in time per
// neuron, parallel over neurons; plus the fused surrogate-gradient pass of its backward.
//
// HBM-bound (12 B per neuron-timestep: read u, write u', write s).  A neuron's row must be
// walked in time order, so one lane owns one neuron; but lanes that each walk their own row in
// global memory would touch 64 different cache lines per access.  Instead a 64-lane work-group
// owns 64 consecutive rows and streams them through LDS in 32-sample time chunks:
//
//   load    : 128-byte row segments, lanes along time (coalesced), written into an LDS ring
//             ring[row][t mod L] that always holds the samples the refractory kernel can
//             still reach (the current chunk plus ceil((nuSize-1)/32) chunks ahead);
//   process : lane = row; for each t of the chunk read ring[row][t], compare with theta and,
//             on a spike, add nu[0..nuSize) onto ring[row][t..t+nuSize) in place - the same
//             fp32 additions in the same order as the sequential loop, hence bit-identical;
//   store   : finished samples leave the ring as 128-byte row segments again; the spikes of a
//             chunk travel as one 32-bit mask per lane and are expanded on the way out.
//
// The ring is rotated by the row number (sample t of row r lives at column (t + r) mod L), so
// both access patterns - a fixed column over 32 rows and 32 consecutive columns of one row -
// hit 32 different LDS banks.
//
// Short refractory kernels (nuSize <= 24, the normal case) use a faster variant of the same
// scheme: the samples the refractory kernel can still reach live in a per-lane register
// window instead of the ring, so the in-place additions are register adds and LDS only
// transposes the chunk on its way in and out.
#include "common.h"

namespace slayer {

constexpr int kSpikeChunk = 32;  // samples per chunk = bits of the per-lane spike mask

// ---- generic kernel: one lane per neuron, in place in global memory (any nuSize) ----------------
__global__ __launch_bounds__(256) void spike_generic_kernel(float *__restrict__ s, float *u,
                                                            const float *__restrict__ nu,
                                                            int64_t rows, int64_t T, int64_t nuSize,
                                                            float theta, float Ts)
{
    const int64_t row = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    const float amplitude = 1.0f / Ts;
    float *ur = u + row * T;
    float *sr = s + row * T;
    for (int64_t t = 0; t < T; ++t) {
        if (ur[t] >= theta) {
            sr[t] = amplitude;
            const int64_t last = (t + nuSize <= T) ? nuSize : (T - t);
            for (int64_t j = 0; j < last; ++j) ur[t + j] += nu[j];
        } else {
            sr[t] = 0.0f;
        }
    }
}

// ---- streaming kernel -------------------------------------------------------------------------------
// L: ring length in samples (power of two); holds (L / 32) chunks per row.
template <int L>
__global__ __launch_bounds__(64) void spike_stream_kernel(float *__restrict__ s, float *u,
                                                          const float *__restrict__ nu,
                                                          int64_t rows, int T, int nuSize,
                                                          float theta, float Ts)
{
    __shared__ float ring[kWave * L];

    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kWave;
    const float amplitude = 1.0f / Ts;
    const int nChunks = (T + kSpikeChunk - 1) / kSpikeChunk;
    const int ahead = (nuSize > 1) ? (nuSize - 2) / kSpikeChunk + 1 : 0;  // chunks of look-ahead

    // lanes-along-time view used by load and store: two row segments per instruction
    const int segT = lane & 31;
    const int segR = lane >> 5;

    auto slot = [](int r, int t) { return r * L + ((t + r) & (L - 1)); };

    auto load_chunk = [&](int c) {
        const int t = c * kSpikeChunk + segT;
#pragma unroll 8
        for (int it = 0; it < 32; ++it) {
            const int r = 2 * it + segR;
            const int64_t row = row0 + r;
            float v = 0.0f;
            if (row < rows && t < T) v = u[row * static_cast<int64_t>(T) + t];
            ring[slot(r, t)] = v;
        }
    };

    for (int c = 0; c < ahead && c < nChunks; ++c) load_chunk(c);

    for (int c = 0; c < nChunks; ++c) {
        if (c + ahead < nChunks) load_chunk(c + ahead);
        __syncthreads();

        // process: lane = row
        uint32_t fired = 0;
        const int tBase = c * kSpikeChunk;
        const int steps = min(kSpikeChunk, T - tBase);
        for (int k = 0; k < steps; ++k) {
            const int t = tBase + k;
            const float x = ring[slot(lane, t)];
            if (x >= theta) {
                fired |= 1u << k;
                const int last = min(nuSize, T - t);
                int j = 0;
                for (; j + 4 <= last; j += 4) {
                    const int i0 = slot(lane, t + j), i1 = slot(lane, t + j + 1);
                    const int i2 = slot(lane, t + j + 2), i3 = slot(lane, t + j + 3);
                    float a0 = ring[i0], a1 = ring[i1], a2 = ring[i2], a3 = ring[i3];
                    a0 += nu[j]; a1 += nu[j + 1]; a2 += nu[j + 2]; a3 += nu[j + 3];
                    ring[i0] = a0; ring[i1] = a1; ring[i2] = a2; ring[i3] = a3;
                }
                for (; j < last; ++j) ring[slot(lane, t + j)] += nu[j];
            }
        }
        __syncthreads();

        // store: finished chunk c leaves the ring
        {
            const int t = tBase + segT;
#pragma unroll 8
            for (int it = 0; it < 32; ++it) {
                const int r = 2 * it + segR;
                const int64_t row = row0 + r;
                const float uv = ring[slot(r, t)];
                const uint32_t m = __shfl(fired, r, kWave);
                const float sv = ((m >> segT) & 1u) ? amplitude : 0.0f;
                if (row < rows && t < T) {
                    const int64_t g = row * static_cast<int64_t>(T) + t;
                    u[g] = uv;
                    s[g] = sv;
                }
            }
        }
        __syncthreads();
    }
}

// ---- register-window kernel (nuSize <= NU) -----------------------------------------------------------
// NU: window length, a compile-time bound on nuSize.  Lane = row keeps v[0 .. 32+NU-2], the
// membrane potential of 32 + NU - 1 consecutive time steps.  Each trip loads the next 32
// samples of every row (transposed through LDS), walks 32 time steps - a spike adds nu[0..NU)
// onto v[k .. k+NU) - and retires the 32 oldest samples.  The walk therefore lags the loads by
// NU - 1 steps.  Taps beyond nuSize are -0.0f, whose addition changes no value; positions
// before the first and after the last sample hold NaN, which never reaches the threshold.
//
// Global traffic uses buffer addressing: one per-lane byte offset (row parity and time within
// the segment) plus a wave-uniform scalar offset per row pair, so the 32 loads of a trip need
// no per-load address registers, are all issued together one trip ahead of their use, and stay
// in flight while the current trip is walked.
template <int NU>
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4, 8))) void spike_window_kernel(
    float *__restrict__ s, float *u, const float *__restrict__ nu, int64_t rows, int T, int nuSize,
    float theta, float Ts)
{
    constexpr int C = kSpikeChunk;
    constexpr int LAG = NU - 1;
    constexpr int P = C + 1;  // padded pitch: column k of row r sits in bank (r + k) mod 32
    __shared__ float tile[kWave * P];

    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kWave;
    const bool fullTile = row0 + kWave <= rows;
    const float amplitude = 1.0f / Ts;
    const float quiet = __builtin_nanf("");
    const int segT = lane & 31;
    const int segR = lane >> 5;
    auto slot = [](int r, int k) { return r * P + k; };

    const BufferRsrc bufU = make_buffer(u + row0 * static_cast<int64_t>(T));
    const BufferRsrc bufS = make_buffer(s + row0 * static_cast<int64_t>(T));
    const int laneOff = (segR * T + segT) * 4;  // byte offset of (row parity, time in segment)
    const int pairStride = 2 * T * 4;           // bytes between row pairs

    float tap[NU];
#pragma unroll
    for (int j = 0; j < NU; ++j) tap[j] = (j < nuSize) ? nu[j] : -0.0f;

    float v[C + LAG];
#pragma unroll
    for (int k = 0; k < LAG; ++k) v[k] = quiet;

    float pre[C];
    auto issue_loads = [&](int tLoad) {
        const int off = laneOff + tLoad * 4;
        if (fullTile && tLoad + C <= T) {
#pragma unroll
            for (int i = 0; i < 32; ++i) pre[i] = buffer_load(bufU, off, i * pairStride);
        } else {
            const bool tOk = tLoad + segT < T;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                pre[i] = quiet;
                if (tOk && row0 + 2 * i + segR < rows) pre[i] = buffer_load(bufU, off, i * pairStride);
            }
        }
    };

    const int trips = (T + LAG + C - 1) / C;
    issue_loads(0);
    for (int it = 0; it < trips; ++it) {
        const int tWalk = it * C - LAG;  // first time step walked (and retired) in this trip

        // transpose the loaded chunk through LDS: lane = row gets its next 32 samples
#pragma unroll
        for (int i = 0; i < 32; ++i) tile[slot(2 * i + segR, segT)] = pre[i];
        __syncthreads();
#pragma unroll
        for (int k = 0; k < C; ++k) v[LAG + k] = tile[slot(lane, k)];
        __syncthreads();
        issue_loads((it + 1) * C);  // past the end of the rows this loads nothing

        // walk 32 time steps
        uint32_t fired = 0;
#pragma unroll
        for (int k = 0; k < C; ++k) {
            if (v[k] >= theta) {
                fired |= 1u << k;
#pragma unroll
                for (int j = 0; j < NU; ++j) v[k + j] += tap[j];
            }
        }

        // retire: the 32 oldest samples are final
#pragma unroll
        for (int k = 0; k < C; ++k) tile[slot(lane, k)] = v[k];
        __syncthreads();
        {
            const int off = laneOff + tWalk * 4;
            if (fullTile && tWalk >= 0 && tWalk + C <= T) {
#pragma unroll 8
                for (int i = 0; i < 32; ++i) {
                    const int r = 2 * i + segR;
                    const float uv = tile[slot(r, segT)];
                    const uint32_t m = __shfl(fired, r, kWave);
                    buffer_store(bufU, off, i * pairStride, uv);
                    buffer_store(bufS, off, i * pairStride, ((m >> segT) & 1u) ? amplitude : 0.0f);
                }
            } else {
                const int t = tWalk + segT;
                const bool tOk = t >= 0 && t < T;
#pragma unroll 8
                for (int i = 0; i < 32; ++i) {
                    const int r = 2 * i + segR;
                    const float uv = tile[slot(r, segT)];
                    const uint32_t m = __shfl(fired, r, kWave);
                    if (tOk && row0 + r < rows) {
                        buffer_store(bufU, off, i * pairStride, uv);
                        buffer_store(bufS, off, i * pairStride, ((m >> segT) & 1u) ? amplitude : 0.0f);
                    }
                }
            }
        }
        __syncthreads();
#pragma unroll
        for (int k = 0; k < LAG; ++k) v[k] = v[C + k];
    }
}

// ---- surrogate gradient ------------------------------------------------------------------------------
template <int VEC>
__global__ __launch_bounds__(256) void spike_bwd_kernel(float *gradIn, const float *gradOut,
                                                        const float *__restrict__ u, float theta,
                                                        float tau, float gain, int64_t numel)
{
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x * VEC;
    for (int64_t i = (static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x) * VEC; i < numel;
         i += stride) {
        if (VEC == 4) {
            const float4 g = *reinterpret_cast<const float4 *>(gradOut + i);
            const float4 x = *reinterpret_cast<const float4 *>(u + i);
            float4 o;
            o.x = g.x * (gain * expf(-fabsf(x.x - theta) / tau));
            o.y = g.y * (gain * expf(-fabsf(x.y - theta) / tau));
            o.z = g.z * (gain * expf(-fabsf(x.z - theta) / tau));
            o.w = g.w * (gain * expf(-fabsf(x.w - theta) / tau));
            *reinterpret_cast<float4 *>(gradIn + i) = o;
        } else {
            gradIn[i] = gradOut[i] * (gain * expf(-fabsf(u[i] - theta) / tau));
        }
    }
}

}  // namespace slayer

extern "C" int slayer_get_spikes_f32(float *s, float *u, const float *nu, int64_t nNeurons,
                                     int64_t T, int64_t nuSize, float theta, float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || nuSize < 0) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !u || (nuSize > 0 && !nu)) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);

    const int64_t groups = ceil_div(nNeurons, kWave);
    const bool stream_ok = !generic_forced() && T < (1LL << 30) && groups < (1LL << 31);
    const bool window_ok = stream_ok && T <= kBufferMaxT;
#define SLAYER_SPIKE_WINDOW(NU)                                                                          \
    do {                                                                                                \
        hipLaunchKernelGGL(spike_window_kernel<NU>, dim3(static_cast<unsigned>(groups)), dim3(kWave), 0,  \
                           st, s, u, nu, nNeurons, static_cast<int>(T), static_cast<int>(nuSize), theta,  \
                           Ts);                                                                         \
        return launch_status();                                                                         \
    } while (0)
    if (window_ok && nuSize <= 24) {
        if (nuSize <= 4) SLAYER_SPIKE_WINDOW(4);
        if (nuSize <= 8) SLAYER_SPIKE_WINDOW(8);
        if (nuSize <= 12) SLAYER_SPIKE_WINDOW(12);
        if (nuSize <= 16) SLAYER_SPIKE_WINDOW(16);
        SLAYER_SPIKE_WINDOW(24);
    }
#undef SLAYER_SPIKE_WINDOW
    if (stream_ok && nuSize <= 33) {
        hipLaunchKernelGGL(spike_stream_kernel<64>, dim3(static_cast<unsigned>(groups)), dim3(kWave), 0,
                           st, s, u, nu, nNeurons, static_cast<int>(T), static_cast<int>(nuSize), theta,
                           Ts);
        return launch_status();
    }
    if (stream_ok && nuSize <= 97) {
        hipLaunchKernelGGL(spike_stream_kernel<128>, dim3(static_cast<unsigned>(groups)), dim3(kWave),
                           0, st, s, u, nu, nNeurons, static_cast<int>(T), static_cast<int>(nuSize),
                           theta, Ts);
        return launch_status();
    }
    const int64_t blocks = ceil_div(nNeurons, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    hipLaunchKernelGGL(spike_generic_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, s, u,
                       nu, nNeurons, T, nuSize, theta, Ts);
    return launch_status();
}

extern "C" int slayer_spike_bwd_f32(float *gradIn, const float *gradOut, const float *u, float theta,
                                    float tau, float scale, int64_t numel, void *stream)
{
    using namespace slayer;
    if (numel < 0) return SLAYER_EINVAL;
    if (numel == 0) return SLAYER_OK;
    if (!gradIn || !gradOut || !u || tau == 0.0f) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const float gain = scale / tau;
    const bool vec4 = (numel % 4 == 0) && aligned16(gradIn) && aligned16(gradOut) && aligned16(u);
    const int64_t perBlock = 256 * (vec4 ? 4 : 1) * 4;  // four trips per lane
    int64_t blocks = ceil_div(numel, perBlock);
    if (blocks > (1LL << 30)) blocks = 1LL << 30;
    if (vec4)
        hipLaunchKernelGGL(spike_bwd_kernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           gradIn, gradOut, u, theta, tau, gain, numel);
    else
        hipLaunchKernelGGL(spike_bwd_kernel<1>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           gradIn, gradOut, u, theta, tau, gain, numel);
    return launch_status();
}

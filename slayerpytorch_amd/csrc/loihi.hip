// Loihi CUBA neuron: int32 current/voltage with sign-magnitude decay (>>12), integer
// threshold, refractory delay.  Sequential in time per neuron, parallel over neurons.
//
// HBM-bound (16 B per neuron-timestep: read w, write spike, voltage, current).  Same streaming
// scheme as the SRM spike kernel: a 64-lane work-group owns 64 consecutive rows and moves them
// through LDS in 32-sample chunks, lanes along time for the 128-byte global segments, lane =
// row for the sequential update.  The neuron state (current, voltage, refractory countdown)
// stays in registers across chunks.  The chunk's input tile is overwritten in place by the
// current; the voltage has its own tile; spikes travel as one 32-bit mask per lane.
//
// Refractory bookkeeping: the sequential formulation keeps a counter that is incremented at a
// spike and decremented refDelay steps later by re-reading the spike it wrote then.  Because a
// spike needs the counter to be zero, the counter only takes the values 0 and 1, and "1" lasts
// exactly until refDelay steps after the spike.  A countdown register set to refDelay at a
// spike and decremented once per step (before the threshold test) is therefore the same
// automaton, without the read-back.
#include "common.h"

namespace slayer {

constexpr int kLoihiChunk = 32;

// sign(x) * ((|x| * (4096 - decay)) >> 12) in 32-bit wrap-around arithmetic
__device__ __forceinline__ uint32_t loihi_decay(int x, uint32_t keep)
{
    const uint32_t ux = static_cast<uint32_t>(x);
    const uint32_t mag = (x >= 0) ? ux : (0u - ux);
    const uint32_t scaled = (mag * keep) >> 12;
    return (x >= 0) ? scaled : (0u - scaled);
}

struct LoihiState {
    int current;
    int voltage;
    uint32_t countdown;  // steps until the neuron may spike again (0 = not refractory)
};

struct LoihiParams {
    uint32_t weightScale, keepI, keepV, refDelay, vDecay;
    int theta;
};

// One time step (t >= 1).  Returns the spike; cOut / vOut are the reported current / voltage.
__device__ __forceinline__ uint32_t loihi_step(LoihiState &st, const LoihiParams &p, float w,
                                               float &cOut, float &vOut)
{
    const int cNew = static_cast<int>(loihi_decay(st.current, p.keepI) +
                                      p.weightScale * static_cast<uint32_t>(trunc_sat(w)));
    const int vNew = static_cast<int>(loihi_decay(st.voltage, p.keepV) + static_cast<uint32_t>(cNew));
    if (st.countdown > 0) --st.countdown;
    const bool refractory = st.countdown != 0;
    const uint32_t spike = (vNew > p.theta && !refractory) ? 1u : 0u;
    st.voltage = (spike || refractory) ? 0 : vNew;
    if (spike) st.countdown = p.refDelay;
    st.current = cNew;
    cOut = static_cast<float>(cNew);
    vOut = spike ? static_cast<float>(static_cast<int>(p.vDecay)) : static_cast<float>(st.voltage);
    return spike;
}

// ---- generic kernel: one lane per neuron, straight from global memory ---------------------------
__global__ __launch_bounds__(256) void loihi_generic_kernel(float *__restrict__ s, float *__restrict__ v,
                                                            float *__restrict__ u,
                                                            const float *__restrict__ w, int64_t rows,
                                                            int64_t T, LoihiParams p)
{
    const int64_t row = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (row >= rows) return;
    const int64_t base = row * T;
    LoihiState st = {0, 0, 0u};
    s[base] = 0.0f; v[base] = 0.0f; u[base] = 0.0f;
    for (int64_t t = 1; t < T; ++t) {
        float c, vo;
        const uint32_t spike = loihi_step(st, p, w[base + t], c, vo);
        s[base + t] = static_cast<float>(spike);
        u[base + t] = c;
        v[base + t] = vo;
    }
}

// ---- streaming kernel -------------------------------------------------------------------------------
// Global traffic uses buffer addressing (per-lane offset + wave-uniform offset per row pair); the
// 32 loads of a chunk are issued one chunk ahead and stay in flight during the sequential update.
__global__ __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(2, 8))) void loihi_stream_kernel(
    float *__restrict__ s, float *__restrict__ v, float *__restrict__ u, const float *__restrict__ w,
    int64_t rows, int T, LoihiParams p)
{
    constexpr int C = kLoihiChunk;
    constexpr int P = C + 1;  // padded pitch: column k of row r sits in bank (r + k) mod 32
    __shared__ float tileC[kWave * P];  // input, then current
    __shared__ float tileV[kWave * P];  // voltage

    const int lane = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kWave;
    const bool fullTile = row0 + kWave <= rows;
    const int nChunks = (T + C - 1) / C;
    const int segT = lane & 31;
    const int segR = lane >> 5;
    auto slot = [](int r, int k) { return r * P + k; };

    const int64_t tileBase = row0 * static_cast<int64_t>(T);
    const BufferRsrc bufW = make_buffer(w + tileBase);
    const BufferRsrc bufS = make_buffer(s + tileBase);
    const BufferRsrc bufV = make_buffer(v + tileBase);
    const BufferRsrc bufU = make_buffer(u + tileBase);
    const int laneOff = (segR * T + segT) * 4;
    const int pairStride = 2 * T * 4;

    float pre[C];
    auto issue_loads = [&](int tBase) {
        const int off = laneOff + tBase * 4;
        if (fullTile && tBase + C <= T) {
#pragma unroll
            for (int i = 0; i < 32; ++i) pre[i] = buffer_load(bufW, off, i * pairStride);
        } else {
            const bool tOk = tBase + segT < T;
#pragma unroll
            for (int i = 0; i < 32; ++i) {
                pre[i] = 0.0f;
                if (tOk && row0 + 2 * i + segR < rows) pre[i] = buffer_load(bufW, off, i * pairStride);
            }
        }
    };

    LoihiState st = {0, 0, 0u};

    issue_loads(0);
    for (int c = 0; c < nChunks; ++c) {
        const int tBase = c * C;
#pragma unroll
        for (int i = 0; i < 32; ++i) tileC[slot(2 * i + segR, segT)] = pre[i];
        __syncthreads();
        issue_loads(tBase + C);  // past the end of the rows this loads nothing

        // sequential update: lane = row
        uint32_t fired = 0;
        const int first = (c == 0) ? 1 : 0;  // t = 0 is forced to zero
        if (c == 0) {
            tileC[slot(lane, 0)] = 0.0f;
            tileV[slot(lane, 0)] = 0.0f;
        }
#pragma unroll 8
        for (int k = first; k < C; ++k) {
            const int i = slot(lane, k);
            float cOut, vOut;
            const uint32_t spike = loihi_step(st, p, tileC[i], cOut, vOut);
            fired |= spike << k;
            tileC[i] = cOut;
            tileV[i] = vOut;
        }
        __syncthreads();

        {
            const int off = laneOff + tBase * 4;
            const bool fast = fullTile && tBase + C <= T;
            const bool tOk = tBase + segT < T;
#pragma unroll 8
            for (int i = 0; i < 32; ++i) {
                const int r = 2 * i + segR;
                const float cv = tileC[slot(r, segT)];
                const float vv = tileV[slot(r, segT)];
                const uint32_t m = __shfl(fired, r, kWave);
                const float sv = ((m >> segT) & 1u) ? 1.0f : 0.0f;
                if (fast || (tOk && row0 + r < rows)) {
                    buffer_store(bufS, off, i * pairStride, sv);
                    buffer_store(bufV, off, i * pairStride, vv);
                    buffer_store(bufU, off, i * pairStride, cv);
                }
            }
        }
        __syncthreads();
    }
}

}  // namespace slayer

extern "C" int slayer_loihi_get_spikes_f32(float *s, float *v, float *u, const float *w,
                                           int64_t nNeurons, int64_t T, uint32_t wgtExp, int32_t theta,
                                           uint32_t iDecay, uint32_t vDecay, uint32_t refDelay,
                                           void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0) return SLAYER_EINVAL;
    if (refDelay == 0 || wgtExp > 25) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !v || !u || !w) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);

    LoihiParams p;
    p.weightScale = 1u << (6 + wgtExp);
    p.keepI = 4096u - iDecay;
    p.keepV = 4096u - vDecay;
    p.refDelay = refDelay;
    p.vDecay = vDecay;
    p.theta = theta;

    const int64_t groups = ceil_div(nNeurons, kWave);
    if (!generic_forced() && T <= kBufferMaxT && groups < (1LL << 31)) {
        hipLaunchKernelGGL(loihi_stream_kernel, dim3(static_cast<unsigned>(groups)), dim3(kWave), 0, st,
                           s, v, u, w, nNeurons, static_cast<int>(T), p);
        return launch_status();
    }
    const int64_t blocks = ceil_div(nNeurons, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    hipLaunchKernelGGL(loihi_generic_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, s, v,
                       u, w, nNeurons, T, p);
    return launch_status();
}

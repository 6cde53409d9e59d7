// PSP filter and spike function in one kernel, for networks that apply them back to back
// (spike(psp(x)), the ordering of the reference's MLP example):
//
//   u[n][t] = Ts * sum_{i<F} a[n][t-i] * srm[i]        (the causal convolution of fir.hip)
//   then the sequential threshold / refractory loop of spike.hip on u, in place.
//
// Same values, bit for bit, as slayer_conv_f32 followed by slayer_get_spikes_f32, without the
// round trip of u through memory: 12 bytes per neuron-timestep (read a, write u', write s)
// instead of 20.  A 64-lane work-group owns 8 whole rows.  It stages them into LDS reversed in
// time and zero padded (X[r][j] = a[r][tHi - j]), runs the register-window FIR core over
// (row, 8-output chunk) items - every lane keeps the results of its items in registers until
// all lanes have finished reading X - then lays the membrane potential out in the same LDS as
// the tile that the spike walk expects (lanes 0..7 walk one row each), and finally stores u'
// and s as whole 16-byte vectors.  Rows must be whole vectors and short enough to travel
// whole; any other shape takes the two separate kernels.
#include "common.h"
#include "fir_core.h"

namespace slayer {

constexpr int kFusedRows = 8;
constexpr int kFusedMaxT = 352;
constexpr int kFusedU = 8;  // outputs per FIR item

template <int NU>
__global__ __launch_bounds__(64) void psp_spike_kernel(float *__restrict__ s, float *__restrict__ u,
                                                       const float *__restrict__ a, const float *__restrict__ srm,
                                                       const float *__restrict__ nu, int64_t rows, int T, int F,
                                                       int nuSize, int LD, int P, int MP, float theta, float Ts)
{
    constexpr int R = kFusedRows, U = kFusedU, G = 32;
    constexpr int LAG = (NU + 2) & ~3;                     // look-ahead of the walk (>= NU - 1, whole vectors)
    constexpr int NBV = R * kFusedMaxT / 4 / kWave;        // vectors per lane of a tile, at most
    constexpr int NIT = (R * (kFusedMaxT / U) + kWave - 1) / kWave;  // FIR items per lane, at most
    extern __shared__ __align__(16) float lds[];
    float *X = lds;                                        // [R][LD] during the FIR ..
    float *tile = lds;                                     // .. then [R][P] for the walk
    uint32_t *masks = reinterpret_cast<uint32_t *>(lds + R * (LD > P ? LD : P));  // [R][MP]

    const int lane = threadIdx.x;
    const int perRow = T >> 2;
    const int ttp = (T + U - 1) & ~(U - 1);                // outputs per row rounded up to whole items
    const int tHi = ttp - 1;                               // time stored at X[.][0]
    const float quiet = __builtin_nanf("");
    const float amplitude = 1.0f / Ts;
    float tap[NU];
#pragma unroll
    for (int j = 0; j < NU; ++j) tap[j] = (j < nuSize) ? nu[j] : -0.0f;

    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), rows - row0));
    const int nVec = nRows * perRow;

    // ---- stage: the tile is one contiguous run of nVec vectors
    float4 x[NBV];
    {
        const BufferRsrc bufA = make_buffer(a + row0 * static_cast<int64_t>(T));
#pragma unroll
        for (int b = 0; b < NBV; ++b)
            x[b] = buffer_load4(bufA, masked_offset(lane + b * kWave < nVec, (lane + b * kWave) * 16), 0);
    }
    for (int i = lane; i < (R * LD) >> 2; i += kWave)
        reinterpret_cast<float4 *>(X)[i] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    wave_sync();
    {
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NBV; ++b) {
            if (lane + b * kWave < nVec)  // times 4c .. 4c+3 land mirrored at columns tHi-4c-3 .. tHi-4c
                *reinterpret_cast<float4 *>(X + rc.r * LD + (tHi - (rc.c << 2) - 3)) =
                    make_float4(x[b].w, x[b].z, x[b].y, x[b].x);
            rc.advance(dr, dc, perRow);
        }
    }
    wave_sync();

    // ---- FIR: item = (row, chunk of U outputs); Y[m] = sum_i X[m+i] * srm[i] is the output at time tHi - m
    const int nChunks = ttp / U;
    const int items = nRows * nChunks;
    float res[NIT][U];
    {
        RowCol item;
        item.init(lane, nChunks, 1.0f / static_cast<float>(nChunks));
        const int dr = kWave / nChunks, dc = kWave % nChunks;
        const int F4 = F & ~3;
        constexpr int NQ = U / 4 + 1;
#pragma unroll
        for (int k = 0; k < NIT; ++k) {
            float acc[U];
#pragma unroll
            for (int j = 0; j < U; ++j) acc[j] = 0.0f;
            if (lane + k * kWave < items) {
                const float4 *xq = reinterpret_cast<const float4 *>(X + item.r * LD + item.c * U);
                float4 q[NQ];
#pragma unroll
                for (int v = 0; v < NQ; ++v) q[v] = xq[v];
                int i = 0, qi = NQ;
                for (; i + 4 * NQ <= F4; i += 4 * NQ, qi += NQ) TripBlocks<U, 0>::run(acc, q, xq, qi, srm + i);
                TailBlocks<U, 0>::run(acc, q, xq, qi, srm + i, F - i);
            }
#pragma unroll
            for (int j = 0; j < U; ++j) res[k][j] = acc[j] * Ts;
            item.advance(dr, dc, nChunks);
        }
    }
    wave_sync();  // every lane is done with X: its memory becomes the tile

    // ---- lay out the membrane potential: tile[r][LAG + t]
    {
        RowCol item;
        item.init(lane, nChunks, 1.0f / static_cast<float>(nChunks));
        const int dr = kWave / nChunks, dc = kWave % nChunks;
#pragma unroll
        for (int k = 0; k < NIT; ++k) {
            if (lane + k * kWave < items) {
                const int tl = tHi - item.c * U - (U - 1);  // lowest time of the chunk, a multiple of U
                float *dst = tile + item.r * P + LAG + tl;
#pragma unroll
                for (int v = 0; v < U / 4; ++v)
                    if (tl + 4 * v < T)  // T is a multiple of 4: a vector is all in or all out
                        *reinterpret_cast<float4 *>(dst + 4 * v) =
                            make_float4(res[k][U - 1 - 4 * v], res[k][U - 2 - 4 * v], res[k][U - 3 - 4 * v],
                                        res[k][U - 4 - 4 * v]);
            }
            item.advance(dr, dc, nChunks);
        }
    }
    wave_sync();

    // ---- walk: lane = row, 32 samples at a time through a register window (see spike.hip)
    const int W = T + LAG;
    if (lane < R) {
        float v[G + LAG];
        float *mine = tile + lane * P;
#pragma unroll
        for (int k = 0; k < LAG; ++k) v[k] = quiet;
        const int groups = (W + G - 1) / G;
        for (int g = 0; g < groups; ++g) {
            const int c0 = g * G;
            if (c0 + G <= T) {
#pragma unroll
                for (int k = 0; k < G; k += 4) {
                    const float4 q = *reinterpret_cast<const float4 *>(mine + LAG + c0 + k);
                    v[LAG + k] = q.x; v[LAG + k + 1] = q.y; v[LAG + k + 2] = q.z; v[LAG + k + 3] = q.w;
                }
            } else {
#pragma unroll
                for (int k = 0; k < G; ++k) v[LAG + k] = (c0 + k < T) ? mine[LAG + c0 + k] : quiet;
            }
            uint32_t fired = 0;
#pragma unroll
            for (int k = 0; k < G; k += 2) {  // one scalar branch per two samples, as in spike.hip
                if (__builtin_amdgcn_ballot_w64((v[k] >= theta) | (v[k + 1] >= theta)) != 0) {
                    if (v[k] >= theta) {
                        fired |= 1u << k;
#pragma unroll
                        for (int j = 0; j < NU; ++j) v[k + j] += tap[j];
                    }
                    if (v[k + 1] >= theta) {
                        fired |= 2u << k;
#pragma unroll
                        for (int j = 0; j < NU; ++j) v[k + 1 + j] += tap[j];
                    }
                }
            }
#pragma unroll
            for (int k = 0; k < G; k += 4)
                *reinterpret_cast<float4 *>(mine + c0 + k) = make_float4(v[k], v[k + 1], v[k + 2], v[k + 3]);
            masks[lane * MP + g] = fired;
#pragma unroll
            for (int k = 0; k < LAG; ++k) v[k] = v[G + k];
        }
    }
    wave_sync();

    // ---- retire: u' and s of the whole tile, one contiguous run
    {
        const BufferRsrc bufU = make_buffer(u + row0 * static_cast<int64_t>(T));
        const BufferRsrc bufS = make_buffer(s + row0 * static_cast<int64_t>(T));
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll 4
        for (int g0 = lane; g0 < nVec; g0 += kWave) {
            const int col = LAG + (rc.c << 2);
            const uint32_t m = masks[rc.r * MP + (col >> 5)] >> (col & 31);
            buffer_store4(bufU, g0 * 16, 0, *reinterpret_cast<const float4 *>(tile + rc.r * P + col));
            buffer_store4(bufS, g0 * 16, 0,
                          make_float4((m & 1u) ? amplitude : 0.0f, (m & 2u) ? amplitude : 0.0f,
                                      (m & 4u) ? amplitude : 0.0f, (m & 8u) ? amplitude : 0.0f));
            rc.advance(dr, dc, perRow);
        }
    }
}

}  // namespace slayer

extern "C" int slayer_psp_spike_f32(float *s, float *u, const float *a, const float *srm, const float *nu,
                                    int64_t nNeurons, int64_t T, int64_t F, int64_t nuSize, float theta,
                                    float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || F < 0 || nuSize < 0) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !u || !a || (F > 0 && !srm) || (nuSize > 0 && !nu)) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);

    const int64_t tiles = ceil_div(nNeurons, kFusedRows);
    const bool fused = !generic_forced() && T % 4 == 0 && T <= kFusedMaxT && F >= 1 && F <= 160 && nuSize <= 24 &&
                       aligned16(s) && aligned16(u) && aligned16(a) && tiles < (1LL << 31);
    if (!fused) {  // the two kernels, one after the other
        const int status = slayer_conv_f32(u, a, srm, nNeurons, T, F, Ts, stream);
        if (status != SLAYER_OK) return status;
        return slayer_get_spikes_f32(s, u, nu, nNeurons, T, nuSize, theta, Ts, stream);
    }
    const int ttp = static_cast<int>((T + kFusedU - 1) & ~static_cast<int64_t>(kFusedU - 1));
    const int LD = static_cast<int>((ttp + F + 4 + 3) & ~static_cast<int64_t>(3));  // tile, halo, window over-read
#define SLAYER_PSP_SPIKE(NU)                                                                                  \
    do {                                                                                                     \
        constexpr int LAG = (NU + 2) & ~3;                                                                   \
        const int cols = (LAG + static_cast<int>(T) + 31) & ~31;                                             \
        const int P = cols + 4, MP = cols / 32 + 1;                                                          \
        const size_t lds = (static_cast<size_t>(kFusedRows) * (LD > P ? LD : P) + kFusedRows * MP) * sizeof(float); \
        hipLaunchKernelGGL((psp_spike_kernel<NU>), dim3(static_cast<unsigned>(tiles)), dim3(kWave), lds, st, s, u, \
                           a, srm, nu, nNeurons, static_cast<int>(T), static_cast<int>(F),                   \
                           static_cast<int>(nuSize), LD, P, MP, theta, Ts);                                  \
        return launch_status();                                                                              \
    } while (0)
    if (nuSize <= 4) SLAYER_PSP_SPIKE(4);
    if (nuSize <= 8) SLAYER_PSP_SPIKE(8);
    if (nuSize <= 12) SLAYER_PSP_SPIKE(12);
    if (nuSize <= 16) SLAYER_PSP_SPIKE(16);
    SLAYER_PSP_SPIKE(24);
#undef SLAYER_PSP_SPIKE
}

// Temporal FIR of neuron rows: causal convolution (PSP forward) and anti-causal correlation
// (PSP backward) with one filter shared by all rows.
//
//   conv: out[n][t] = Ts * sum_i in[n][t-i] * filt[i]     corr: out[n][t] = Ts * sum_i in[n][t+i] * filt[i]
//
// Every output is one chain acc = fma(in, filt[i], acc) over i = 0,1,..,F-1 starting from 0,
// then one multiply by Ts, exactly like the sequential loop; samples outside [0,T) enter as
// zeros, which leaves the chain's value unchanged.
//
// Tiled kernel.  The convolution is the correlation on a reversed time axis, so both share one
// core: Y[m] = sum_i X[m+i] * filt[i].  A work-group of 256 lanes owns 32 neuron rows and one
// time tile; it stages the rows' samples (plus the F-1 sample halo) into LDS as X[32][LD]
// (reversed for the convolution).  Lane l works on row (l & 31); each half-wave is one "slot"
// that takes 8-output chunks of the tile.  A lane keeps a 12-sample register window of X and
// slides it 4 samples per 4 taps with one 16-byte LDS read, so one LDS read feeds 32 FMAs;
// LD = 4 (mod 32) makes those reads bank-conflict free across the 32 rows of a slot.  Filter
// taps are wave-uniform and come through scalar loads.  An FIR with F = 77 taps needs 154
// flop per 8 bytes moved, which is at the FP32 ridge of the machine: the kernel is built to
// be FMA-issue bound, not LDS or HBM bound.
#include "common.h"

namespace slayer {

constexpr int kFirRows = 32;    // rows per work-group
constexpr int kFirSlots = 8;    // half-waves per work-group
constexpr int kFirU = 8;        // outputs per lane per chunk
constexpr int kFirMaxLD = 388;  // LDS row pitch limit: 32*388*4 B = 48.5 KiB, three groups per CU

// ---- generic kernel: one lane per output sample (any F, any T) ---------------------------------
template <bool CAUSAL>
__global__ __launch_bounds__(256) void fir_generic_kernel(float *__restrict__ out,
                                                          const float *__restrict__ in,
                                                          const float *__restrict__ filt,
                                                          int64_t rows, int64_t T, int64_t F, float Ts)
{
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= T) return;
    for (int64_t row = blockIdx.y; row < rows; row += gridDim.y) {
        const float *x = in + row * T;
        float acc = 0.0f;
        if (CAUSAL) {
            const int64_t taps = (t + 1 < F) ? (t + 1) : F;
            for (int64_t i = 0; i < taps; ++i) acc = __builtin_fmaf(x[t - i], filt[i], acc);
        } else {
            const int64_t taps = (T - t < F) ? (T - t) : F;
            for (int64_t i = 0; i < taps; ++i) acc = __builtin_fmaf(x[t + i], filt[i], acc);
        }
        out[row * T + t] = acc * Ts;
    }
}

// ---- tiled kernel ---------------------------------------------------------------------------------
__device__ __forceinline__ void fma_quad(float (&acc)[kFirU], const float4 &a, const float4 &b,
                                         const float4 &c, float f0, float f1, float f2, float f3)
{
    // window w[0..11] = (a, b, c); output j, tap s uses w[j + s]
    const float w[12] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w, c.x, c.y, c.z, c.w};
#pragma unroll
    for (int j = 0; j < kFirU; ++j) {
        acc[j] = __builtin_fmaf(w[j + 0], f0, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 1], f1, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 2], f2, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 3], f3, acc[j]);
    }
}

template <bool CAUSAL>
__global__ __launch_bounds__(256) void fir_tiled_kernel(float *__restrict__ out,
                                                        const float *__restrict__ in,
                                                        const float *__restrict__ filt,
                                                        int64_t rows, int T, int F, int TT, int LD,
                                                        float Ts)
{
    extern __shared__ __align__(16) float X[];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * kFirRows;
    const int t0 = blockIdx.y * TT;                 // first output time of the tile
    const int tt = min(TT, T - t0);                 // outputs in this tile
    const int ttp = (tt + kFirU - 1) & ~(kFirU - 1);  // rounded up to whole chunks
    const int tHi = t0 + ttp - 1;                   // time stored at X[.][0] when reversed
    const int used = ttp + F + 4;                   // samples of a row the core may read

    // stage: X[r][j] = in[row0+r][time(j)], zero outside the row; time(j) = t0+j (corr) or tHi-j (conv)
    for (int r = wave; r < kFirRows; r += 4) {
        const int64_t row = row0 + r;
        const float *src = in + row * static_cast<int64_t>(T);
        float *dst = X + r * LD;
        for (int j = lane; j < used; j += kWave) {
            const int time = CAUSAL ? (tHi - j) : (t0 + j);
            float v = 0.0f;
            if (row < rows && time >= 0 && time < T) v = src[time];
            dst[j] = v;
        }
    }
    __syncthreads();

    const int r = lane & 31;
    const int slot = wave * 2 + (lane >> 5);
    const int64_t row = row0 + r;
    const float *xr = X + r * LD;
    const int nChunks = ttp / kFirU;
    const int F4 = F & ~3;

    for (int c = slot; c < nChunks; c += kFirSlots) {
        const int m0 = c * kFirU;
        float acc[kFirU];
#pragma unroll
        for (int j = 0; j < kFirU; ++j) acc[j] = 0.0f;

        const float4 *xq = reinterpret_cast<const float4 *>(xr + m0);
        float4 qa = xq[0], qb = xq[1], qc = xq[2];
        int i = 0, q = 3;
        // three 4-tap blocks per trip so that the window rotates through registers without moves
        for (; i + 12 <= F4; i += 12, q += 3) {
            fma_quad(acc, qa, qb, qc, filt[i], filt[i + 1], filt[i + 2], filt[i + 3]);
            qa = xq[q];
            fma_quad(acc, qb, qc, qa, filt[i + 4], filt[i + 5], filt[i + 6], filt[i + 7]);
            qb = xq[q + 1];
            fma_quad(acc, qc, qa, qb, filt[i + 8], filt[i + 9], filt[i + 10], filt[i + 11]);
            qc = xq[q + 2];
        }
        if (i + 4 <= F4) {
            fma_quad(acc, qa, qb, qc, filt[i], filt[i + 1], filt[i + 2], filt[i + 3]);
            const float4 n = xq[q];
            qa = qb; qb = qc; qc = n;
            i += 4; ++q;
        }
        if (i + 4 <= F4) {
            fma_quad(acc, qa, qb, qc, filt[i], filt[i + 1], filt[i + 2], filt[i + 3]);
            const float4 n = xq[q];
            qa = qb; qb = qc; qc = n;
            i += 4; ++q;
        }
        if (i < F) {  // 1..3 remaining taps
            const float f0 = filt[i];
            const float f1 = (i + 1 < F) ? filt[i + 1] : 0.0f;
            const float f2 = (i + 2 < F) ? filt[i + 2] : 0.0f;
            const float w[12] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w, qc.x, qc.y, qc.z, qc.w};
#pragma unroll
            for (int j = 0; j < kFirU; ++j) {
                acc[j] = __builtin_fmaf(w[j], f0, acc[j]);
                if (i + 1 < F) acc[j] = __builtin_fmaf(w[j + 1], f1, acc[j]);
                if (i + 2 < F) acc[j] = __builtin_fmaf(w[j + 2], f2, acc[j]);
            }
        }

        if (row < rows) {
            float *dst = out + row * static_cast<int64_t>(T);
#pragma unroll
            for (int j = 0; j < kFirU; ++j) {
                const int m = m0 + j;
                const int time = CAUSAL ? (tHi - m) : (t0 + m);
                if (time >= t0 && time < t0 + tt) dst[time] = acc[j] * Ts;
            }
        }
    }
}

template <bool CAUSAL>
static int launch_fir(float *out, const float *in, const float *filt, int64_t rows, int64_t T,
                      int64_t F, float Ts, hipStream_t stream)
{
    if (rows < 0 || T < 0 || F < 0) return SLAYER_EINVAL;
    if (rows == 0 || T == 0) return SLAYER_OK;
    if (!out || !in || (F > 0 && !filt)) return SLAYER_EINVAL;
    if (T >= (1LL << 30)) return SLAYER_EUNSUPPORTED;

    // largest tile (multiple of the chunk) whose row pitch fits the LDS budget
    const int64_t ttMax = (kFirMaxLD - 4 - F) & ~static_cast<int64_t>(kFirU - 1);
    const bool tiled = !generic_forced() && F >= 1 && ttMax >= 64 && rows < (1LL << 31) * kFirRows;
    if (tiled) {
        const int64_t nTiles = ceil_div(T, ttMax);
        int64_t TT = ceil_div(ceil_div(T, nTiles), kFirU) * kFirU;
        if (nTiles == 1) TT = T;
        const int64_t ttp = ceil_div(TT, kFirU) * kFirU;
        int64_t LD = ttp + F + 4;
        LD = ((LD - 4 + 31) / 32) * 32 + 4;  // 4 (mod 32): conflict-free 16-byte reads per slot
        const int64_t rowTiles = ceil_div(rows, kFirRows);
        if (nTiles <= 65535 && LD <= kFirMaxLD) {
            dim3 grid(static_cast<unsigned>(rowTiles), static_cast<unsigned>(nTiles)), block(256);
            const size_t lds = static_cast<size_t>(kFirRows) * LD * sizeof(float);
            hipLaunchKernelGGL(fir_tiled_kernel<CAUSAL>, grid, block, lds, stream, out, in, filt, rows,
                               static_cast<int>(T), static_cast<int>(F), static_cast<int>(TT),
                               static_cast<int>(LD), Ts);
            return launch_status();
        }
    }
    const int64_t tBlocks = ceil_div(T, 256);
    if (tBlocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    dim3 grid(static_cast<unsigned>(tBlocks), static_cast<unsigned>(rows < 65535 ? rows : 65535));
    hipLaunchKernelGGL(fir_generic_kernel<CAUSAL>, grid, dim3(256), 0, stream, out, in, filt, rows, T,
                       F, Ts);
    return launch_status();
}

}  // namespace slayer

extern "C" int slayer_conv_f32(float *out, const float *in, const float *filt, int64_t nNeurons,
                               int64_t T, int64_t F, float Ts, void *stream)
{
    return slayer::launch_fir<true>(out, in, filt, nNeurons, T, F, Ts,
                                    static_cast<hipStream_t>(stream));
}

extern "C" int slayer_corr_f32(float *out, const float *in, const float *filt, int64_t nNeurons,
                               int64_t T, int64_t F, float Ts, void *stream)
{
    return slayer::launch_fir<false>(out, in, filt, nNeurons, T, F, Ts,
                                     static_cast<hipStream_t>(stream));
}

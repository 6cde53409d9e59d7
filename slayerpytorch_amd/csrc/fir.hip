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
// core: Y[m] = sum_i X[m+i] * filt[i].  A work-group of 256 lanes owns R consecutive neuron
// rows and one time tile; it stages the rows' samples (plus the F-1 sample halo, zero padded)
// into LDS as X[R][LD] with 16-byte loads (reversed in time for the convolution).  The tile is
// then cut into chunks of 8 consecutive outputs of one row; lanes take chunks in row-major
// order, so neighbouring lanes produce neighbouring outputs and the results leave as 16-byte
// stores.  A lane keeps a 12-sample register window of X and slides it 4 samples per 4 taps
// with one 16-byte LDS read, i.e. one LDS read feeds 32 FMAs.  Filter taps are wave-uniform
// and come through scalar loads.  An FIR with F = 77 taps needs 154 flop per 8 bytes moved,
// which is at the FP32 ridge of the machine: the kernel is meant to be FMA-issue bound.
#include "common.h"

namespace slayer {

constexpr int kFirU = 8;              // outputs per lane per chunk
constexpr int kFirMaxLdsFloats = 12288;  // 48 KiB of LDS per work-group at most
constexpr int kFirMaxPitch = 512;     // longest LDS row (samples) the tiled kernel stages

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

// VEC: rows are whole 16-byte vectors (T % 4 == 0, pointers 16-byte aligned)
template <bool CAUSAL, bool VEC>
__global__ __launch_bounds__(256) void fir_tiled_kernel(float *__restrict__ out,
                                                        const float *__restrict__ in,
                                                        const float *__restrict__ filt,
                                                        int64_t rows, int T, int F, int TT, int LD, int R,
                                                        float Ts)
{
    extern __shared__ __align__(16) float X[];

    const int tid = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), rows - row0));
    const int t0 = blockIdx.y * TT;                   // first output time of the tile
    const int tt = min(TT, T - t0);                   // outputs in this tile
    const int ttp = (tt + kFirU - 1) & ~(kFirU - 1);  // rounded up to whole chunks
    const int tHi = t0 + ttp - 1;                     // time stored at X[.][0] when reversed
    const int LD4 = LD >> 2;

    // The tile's rows as 32-bit offsets from its first row (a tile spans far less than 2 GiB).
    const BufferRsrc bufIn = make_buffer(in + row0 * static_cast<int64_t>(T));
    const BufferRsrc bufOut = make_buffer(out + row0 * static_cast<int64_t>(T));

    // ---- stage: X[r][j] = in[row0+r][time(j)], zero outside the row;
    //      time(j) = t0 + j (correlation) or tHi - j (convolution)
    if (VEC) {
        // samples of the row that the tile needs: times [tA, tB), whole 16-byte vectors
        const int tA = CAUSAL ? max(0, tHi + 1 - LD) : t0;
        const int tB = CAUSAL ? min(T, tHi + 1) : min(T, t0 + LD);
        const int nq = (tB - tA) >> 2;               // source vectors per row
        const int jA = CAUSAL ? (tHi + 1 - tB) : 0;  // X columns [jA, jA + 4 nq) receive them
        {
            RowCol rc;
            rc.init(tid, nq, 1.0f / static_cast<float>(nq));
            const int dr = 256 / nq, dc = 256 % nq;
            const int total = nRows * nq;
            for (int g = tid; g < total; g += 256, rc.advance(dr, dc, nq)) {
                const float4 v = buffer_load4(bufIn, (rc.r * T + tA + (rc.c << 2)) * 4, 0);
                if (CAUSAL)  // descending time: the vector lands mirrored
                    *reinterpret_cast<float4 *>(X + rc.r * LD + (jA + ((nq - 1 - rc.c) << 2))) =
                        make_float4(v.w, v.z, v.y, v.x);
                else
                    *reinterpret_cast<float4 *>(X + rc.r * LD + (rc.c << 2)) = v;
            }
        }
        // zero padding: columns [0, jA) and [jA + 4 nq, LD)
        const int zq = LD4 - nq;
        if (zq > 0) {
            RowCol rc;
            rc.init(tid, zq, 1.0f / static_cast<float>(zq));
            const int dr = 256 / zq, dc = 256 % zq;
            const int total = nRows * zq;
            const int head = jA >> 2;
            for (int g = tid; g < total; g += 256, rc.advance(dr, dc, zq)) {
                const int j4 = (rc.c < head) ? rc.c : (rc.c + nq);
                *reinterpret_cast<float4 *>(X + rc.r * LD + (j4 << 2)) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            }
        }
    } else {
        const float invLD4 = 1.0f / static_cast<float>(LD4);
        const int quads = nRows * LD4;
        for (int q = tid; q < quads; q += 256) {
            int r, j4;
            divmod_small(q, LD4, invLD4, r, j4);
            const float *src = in + (row0 + r) * static_cast<int64_t>(T);
            const int j = j4 << 2;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            if (CAUSAL) {
                const int tl = tHi - j - 3;  // lowest time of the quad; X order is descending
                if (tl + 3 >= 0 && tl + 3 < T) v.x = src[tl + 3];
                if (tl + 2 >= 0 && tl + 2 < T) v.y = src[tl + 2];
                if (tl + 1 >= 0 && tl + 1 < T) v.z = src[tl + 1];
                if (tl >= 0 && tl < T) v.w = src[tl];
            } else {
                const int tl = t0 + j;
                if (tl < T) v.x = src[tl];
                if (tl + 1 < T) v.y = src[tl + 1];
                if (tl + 2 < T) v.z = src[tl + 2];
                if (tl + 3 < T) v.w = src[tl + 3];
            }
            *reinterpret_cast<float4 *>(X + r * LD + j) = v;
        }
    }
    __syncthreads();

    // ---- compute: work item = (row, chunk of 8 outputs), row-major over lanes
    const int nChunks = ttp / kFirU;
    const int items = nRows * nChunks;
    const int F4 = F & ~3;
    RowCol item;
    item.init(tid, nChunks, 1.0f / static_cast<float>(nChunks));
    const int itemDr = 256 / nChunks, itemDc = 256 % nChunks;

    for (int w = tid; w < items; w += 256, item.advance(itemDr, itemDc, nChunks)) {
        const int r = item.r;
        const int m0 = item.c * kFirU;
        float acc[kFirU];
#pragma unroll
        for (int j = 0; j < kFirU; ++j) acc[j] = 0.0f;

        const float4 *xq = reinterpret_cast<const float4 *>(X + r * LD + m0);
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
            const float wv[12] = {qa.x, qa.y, qa.z, qa.w, qb.x, qb.y, qb.z, qb.w, qc.x, qc.y, qc.z, qc.w};
#pragma unroll
            for (int j = 0; j < kFirU; ++j) {
                acc[j] = __builtin_fmaf(wv[j], f0, acc[j]);
                if (i + 1 < F) acc[j] = __builtin_fmaf(wv[j + 1], f1, acc[j]);
                if (i + 2 < F) acc[j] = __builtin_fmaf(wv[j + 2], f2, acc[j]);
            }
        }

        // ---- store the 8 outputs: times t0+m0 .. +7 (correlation) or tHi-m0-7 .. tHi-m0 (convolution)
        float y[kFirU];
#pragma unroll
        for (int j = 0; j < kFirU; ++j) y[j] = (CAUSAL ? acc[kFirU - 1 - j] : acc[j]) * Ts;
        const int tl = CAUSAL ? (tHi - m0 - (kFirU - 1)) : (t0 + m0);  // lowest time of the chunk
        if (VEC) {
            // tl is a multiple of 4 and so is the tile's end, so each half is all in or all out
            const int off = (r * T + tl) * 4;
            if (tl >= t0 && tl + 3 < t0 + tt) buffer_store4(bufOut, off, 0, make_float4(y[0], y[1], y[2], y[3]));
            if (tl + 4 >= t0 && tl + 7 < t0 + tt)
                buffer_store4(bufOut, off + 16, 0, make_float4(y[4], y[5], y[6], y[7]));
        } else {
            float *dst = out + (row0 + r) * static_cast<int64_t>(T);
#pragma unroll
            for (int j = 0; j < kFirU; ++j)
                if (tl + j >= t0 && tl + j < t0 + tt) dst[tl + j] = y[j];
        }
    }
}

struct FirPlan {
    int TT, LD, R, nTiles;
};

// Chooses the time tile, the LDS row pitch and the rows per work-group.
static bool plan_fir(int64_t rows, int64_t T, int64_t F, FirPlan &p)
{
    // a row of X holds ttp + F + 4 samples (chunk-rounded tile, halo, window over-read)
    const int64_t ttMax = (kFirMaxPitch - 4 - F) & ~static_cast<int64_t>(kFirU - 1);
    if (F < 1 || ttMax < 64 || T > kBufferMaxT) return false;
    const int64_t nTiles = ceil_div(T, ttMax);
    if (nTiles > 65535) return false;
    int64_t TT = ceil_div(ceil_div(T, nTiles), kFirU) * kFirU;
    if (nTiles == 1) TT = T;
    const int64_t ttp = ceil_div(TT, kFirU) * kFirU;
    const int64_t LD = (ttp + F + 4 + 3) & ~static_cast<int64_t>(3);
    const int64_t nChunks = ttp / kFirU;
    // rows per group: fill the 256 lanes evenly with (row, chunk) items, stay within the LDS
    // budget, and prefer small tiles (more groups per CU overlap staging with compute)
    const int64_t rMax = kFirMaxLdsFloats / LD;
    if (rMax < 1) return false;
    int64_t best = 1;
    double bestScore = -1.0;
    for (int64_t r = 1; r <= rMax && r <= 64; ++r) {
        const int64_t items = r * nChunks;
        const double eff = static_cast<double>(items) / static_cast<double>(ceil_div(items, 256) * 256);
        // at least ~3 passes of work per staging, mild preference for less LDS
        const double score = eff - (items < 512 ? 0.25 : 0.0) - 0.02 * static_cast<double>(r * LD) / kFirMaxLdsFloats;
        if (score > bestScore) { bestScore = score; best = r; }
    }
    if (best > rows) best = rows;
    p.TT = static_cast<int>(TT);
    p.LD = static_cast<int>(LD);
    p.R = static_cast<int>(best);
    p.nTiles = static_cast<int>(nTiles);
    return true;
}

template <bool CAUSAL>
static int launch_fir(float *out, const float *in, const float *filt, int64_t rows, int64_t T,
                      int64_t F, float Ts, hipStream_t stream)
{
    if (rows < 0 || T < 0 || F < 0) return SLAYER_EINVAL;
    if (rows == 0 || T == 0) return SLAYER_OK;
    if (!out || !in || (F > 0 && !filt)) return SLAYER_EINVAL;
    if (T >= (1LL << 30)) return SLAYER_EUNSUPPORTED;

    FirPlan p;
    if (!generic_forced() && plan_fir(rows, T, F, p)) {
        const int64_t rowTiles = ceil_div(rows, p.R);
        if (rowTiles < (1LL << 31)) {
            dim3 grid(static_cast<unsigned>(rowTiles), static_cast<unsigned>(p.nTiles)), block(256);
            const size_t lds = static_cast<size_t>(p.R) * p.LD * sizeof(float);
            const bool vec = (T % 4 == 0) && aligned16(out) && aligned16(in);
            if (vec)
                hipLaunchKernelGGL((fir_tiled_kernel<CAUSAL, true>), grid, block, lds, stream, out, in, filt,
                                   rows, static_cast<int>(T), static_cast<int>(F), p.TT, p.LD, p.R, Ts);
            else
                hipLaunchKernelGGL((fir_tiled_kernel<CAUSAL, false>), grid, block, lds, stream, out, in, filt,
                                   rows, static_cast<int>(T), static_cast<int>(F), p.TT, p.LD, p.R, Ts);
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

// Temporal FIR of neuron rows: causal convolution (PSP forward) and anti-causal correlation
// (PSP backward) with one filter shared by all rows.
//
//   conv: out[n][t] = Ts * sum_i in[n][t-i] * filt[i]     corr: out[n][t] = Ts * sum_i in[n][t+i] * filt[i]
//
// The reference's definition of an output is one chain acc = fma(in, filt[i], acc) over i = 0,1,..,F-1
// starting from 0, then one multiply by Ts; samples outside [0,T) enter as zeros, which leaves the
// chain's value unchanged.
//
// Three kernels here (the plain correlation with 34 to 129 taps on rows of whole 16-byte vectors goes to
// the matrix-core kernel of fir_mfma.hip first):
//  * direct: rows of whole 16-byte vectors and filters of at most 33 taps: everything in registers,
//    addressing of a plain copy, the chain bit for bit;
//  * tiled: the convolution is the correlation on a reversed time axis, so both share one core
//    Y[m] = sum_i X[m+i] * filt[i].  A work-group of 256 lanes owns R consecutive neuron rows
//    and one time tile; it stages the rows' samples (plus the F-1 sample halo, zero padded) into
//    LDS as X[R][LD] with 16-byte loads (reversed in time for the convolution) and counts the non-zero
//    samples on the way.  Then one of three paths per tile:
//      - almost all zeros (spike trains): event-driven, one update per non-zero sample, the bits of the
//        chain with its zero terms left out;
//      - dense, 34 to 129 taps, whole-vector rows (template DM > 0): the tile's outputs as products of
//        a banded Toeplitz matrix of the filter with blocks of 16 samples on the matrix cores
//        (v_mfma_f32_16x16x4_f32; fir_core.h has the formulation): agrees with the chain to rounding,
//        a tile with a non-finite sample is recomputed as chains so that infinities and NaNs land
//        where the reference puts them;
//      - otherwise the chain on the vector ALUs: chunks of U (8 or 16) consecutive outputs of one row
//        per lane, a (U+4)-sample register window slid 4 samples per 4 taps with one 16-byte LDS read,
//        taps through scalar loads; bit-identical to the sequential loop.  An FIR with F = 77 taps
//        needs 154 flop per 8 bytes moved, the FP32 ridge of the machine: this path is FMA-issue bound;
//  * generic: one lane per output, any shape.
#include "common.h"
#include "fir_core.h"

namespace slayer {

constexpr int kFirMaxLdsFloats = 12288;  // 48 KiB of LDS per work-group at most
constexpr int kFirMaxPitch = 512;     // longest LDS row (samples) the tiled kernel stages

// four floats that need not be 16-byte aligned (the GPU's global memory accesses may be unaligned)
typedef float float4u __attribute__((ext_vector_type(4), aligned(4)));

// ---- generic kernel: one lane per output sample (any F, any T) ---------------------------------
template <bool CAUSAL, bool GATED>
__global__ __launch_bounds__(256) void fir_generic_kernel(float *__restrict__ out,
                                                          const float *__restrict__ in,
                                                          const float *__restrict__ filt,
                                                          int64_t rows, int64_t T, int64_t F, float Ts, FirGate gate)
{
    const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (t >= T) return;
    for (int64_t row = blockIdx.y; row < rows; row += gridDim.y) {
        const float *x = in + row * T;
        const float *gu = GATED ? gate.u + row * T : nullptr;
        auto sample = [&](int64_t k) {
            return GATED ? x[k] * spike_pdf(gu[k], gate.theta, gate.tau, gate.gain) : x[k];
        };
        float acc = 0.0f;
        if (CAUSAL) {
            const int64_t taps = (t + 1 < F) ? (t + 1) : F;
            for (int64_t i = 0; i < taps; ++i) acc = __builtin_fmaf(sample(t - i), filt[i], acc);
        } else {
            const int64_t taps = (T - t < F) ? (T - t) : F;
            for (int64_t i = 0; i < taps; ++i) acc = __builtin_fmaf(sample(t + i), filt[i], acc);
        }
        out[row * T + t] = acc * Ts;
    }
}

// ---- direct kernel: rows of whole 16-byte vectors, everything in registers -----------------------------
// Lane g of the grid owns a chunk of U consecutive outputs of one row (U/4 aligned 16-byte
// vectors), reads the NV aligned input vectors that hold its U + F - 1 samples straight from
// global memory (neighbouring lanes share them through the caches), runs the U tap chains in
// registers and streams its results out.  No LDS, no barriers; the addressing is that of a plain
// copy.  NV >= (F - 1 + U) / 4.
template <bool CAUSAL, int NV, int U>
__global__ __launch_bounds__(256) void fir_direct_kernel(float *__restrict__ out, const float *__restrict__ in,
                                                         const float *__restrict__ filt, uint32_t chunks, int T,
                                                         int F, FastDiv byRow, float Ts)
{
    constexpr int UV = U / 4;
    const int perRow = T >> 2;                    // vectors per row
    const int chunksPerRow = (perRow + UV - 1) / UV;
    const uint32_t g0 = blockIdx.x * 256u;
    const uint32_t g = g0 + threadIdx.x;
    const bool active = g < chunks;
    const uint32_t rowBase = fastdiv(g0, byRow);  // wave-uniform: addressing is relative to this row
    const uint32_t row = fastdiv(active ? g : g0, byRow);
    const int c = static_cast<int>((active ? g : g0) - row * static_cast<uint32_t>(chunksPerRow));
    const int r = static_cast<int>(row - rowBase);
    const BufferRsrc bufIn = make_buffer(in + static_cast<int64_t>(rowBase) * T);
    const BufferRsrc bufOut = make_buffer(out + static_cast<int64_t>(rowBase) * T);

    // window w[k] = sample 4 * first + k of the row, zero outside the row
    const int first = CAUSAL ? UV * c + UV - NV : UV * c;
    float w[4 * NV];
#pragma unroll
    for (int v = 0; v < NV; ++v) {
        const int qv = first + v;
        const float4 x = buffer_load4<0>(bufIn, masked_offset(active && qv >= 0 && qv < perRow, (r * T + (qv << 2)) * 4), 0);
        w[4 * v] = x.x; w[4 * v + 1] = x.y; w[4 * v + 2] = x.z; w[4 * v + 3] = x.w;
    }
    // all loads are issued before the first tap: keep them from sinking into the tap blocks
#pragma unroll
    for (int k = 0; k < 4 * NV; ++k) asm volatile("" : "+v"(w[k]));

    float acc[U];
#pragma unroll
    for (int e = 0; e < U; ++e) acc[e] = 0.0f;
    constexpr int FMAX = 4 * NV - U + 1;          // longest filter this window serves
    constexpr int B = 8;                          // taps per block
#pragma unroll
    for (int ib = 0; ib < FMAX; ib += B) {
        if (ib + B <= F) {
            float f[B];
#pragma unroll
            for (int k = 0; k < B; ++k) f[k] = filt[ib + k];
#pragma unroll
            for (int k = 0; k < B; ++k) {
                const int i = ib + k;
                if (i < FMAX) {
#pragma unroll
                    for (int e = 0; e < U; ++e)
                        acc[e] = __builtin_fmaf(CAUSAL ? w[4 * NV - U + e - i] : w[e + i], f[k], acc[e]);
                }
            }
        } else {
#pragma unroll
            for (int k = 0; k < B; ++k) {
                const int i = ib + k;
                if (i < FMAX && i < F) {
                    const float fi = filt[i];
#pragma unroll
                    for (int e = 0; e < U; ++e)
                        acc[e] = __builtin_fmaf(CAUSAL ? w[4 * NV - U + e - i] : w[e + i], fi, acc[e]);
                }
            }
        }
    }
    // with several vectors per lane one store instruction leaves gaps that the lane's next store
    // fills: those go through the cache, which merges them into whole memory lines
#pragma unroll
    for (int v = 0; v < UV; ++v)
        buffer_store4<(UV > 1 ? 0 : kStream)>(bufOut, masked_offset(active && UV * c + v < perRow, (r * T + ((UV * c + v) << 2)) * 4), 0,
                      make_float4(acc[4 * v] * Ts, acc[4 * v + 1] * Ts, acc[4 * v + 2] * Ts, acc[4 * v + 3] * Ts));
}

// ---- tiled kernel ---------------------------------------------------------------------------------
// (the register-window core, window_of .. TailBlocks, is in fir_core.h)
// Non-zero samples ("events", low 16 bits) and non-zero vectors (high 16 bits) among the wavefront's vectors;
// non-zero is anything but +0 and -0, by class (denormals and NaNs count).  A tile stages at most 12288 samples,
// so sums of these over a tile stay within their 16 bits.
__device__ __forceinline__ uint32_t count_nonzero(const float4 &v)
{
    constexpr int kNotZero = 0x3ff & ~0x60;  // every class but the two zeros
    const uint64_t mx = __ballot(__builtin_amdgcn_classf(v.x, kNotZero)), my = __ballot(__builtin_amdgcn_classf(v.y, kNotZero));
    const uint64_t mz = __ballot(__builtin_amdgcn_classf(v.z, kNotZero)), mw = __ballot(__builtin_amdgcn_classf(v.w, kNotZero));
    const uint32_t events = __builtin_popcountll(mx) + __builtin_popcountll(my) + __builtin_popcountll(mz) + __builtin_popcountll(mw);
    return events + (static_cast<uint32_t>(__builtin_popcountll(mx | my | mz | mw)) << 16);
}

// ---- event-driven path for sparse input (spike trains) -------------------------------------------
// When few samples of a tile are non-zero, walking the taps wastes almost all of its multiply-adds
// on zeros.  Here a wavefront takes one row at a time, finds the row's non-zero samples ("events")
// with ballots, and for each block of 64 outputs adds the events that can reach it, in ascending
// order of their column: for output m the terms X[j] * filt[j - m] arrive in ascending j, i.e. in
// ascending tap order, which is exactly the dense chain with its zero terms left out - and adding
// a zero term never changes a finite sum - so both paths give the same bits.  All control flow is
// wave-uniform (the event list lives in scalar registers).
constexpr int kSparseBlocks = 7;   // 64-column blocks of an LDS row the sparse path handles (LD <= 448)
constexpr int kSparseMaxTaps = 129;  // an event reaches at most three 64-output blocks

template <bool CAUSAL>
__device__ __forceinline__ void fir_sparse_tile(const BufferRsrc &bufOut, const float *X, const float *fL,
                                                int nRows, int LD, int ttp, int t0, int tt, int tHi, int T,
                                                int F, float Ts)
{
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int nPass = (ttp + kWave - 1) / kWave;  // blocks of 64 outputs; lane's output in block k is 64 k + lane
    for (int r = wave; r < nRows; r += 4) {
        const float *xr = X + r * LD;
        float acc[kSparseBlocks];
#pragma unroll
        for (int k = 0; k < kSparseBlocks; ++k) acc[k] = 0.0f;
        float xb[kSparseBlocks];  // the row, 64 columns per register
#pragma unroll
        for (int b = 0; b < kSparseBlocks; ++b) xb[b] = (b * kWave + lane < LD) ? xr[b * kWave + lane] : 0.0f;
        // events in ascending column order, 64 columns at a time
#pragma unroll
        for (int b = 0; b < kSparseBlocks; ++b) {
            if (b * kWave >= LD) break;
            const float v = xb[b];
            uint64_t mask = __ballot(v != 0.0f);
            while (mask) {
                const int pos = __builtin_ctzll(mask);
                mask &= mask - 1;
                const int xbits = __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), pos);
                const float xv = __builtin_bit_cast(float, xbits);
                // column j = 64 b + pos is tap i = j - m of output m; it reaches the output blocks
                // b, b-1 and b-2 (F <= 129) through the taps i_d = 64 d + pos - lane, d = 0, 1, 2.
                // The filter copy is zero padded on both sides, so the three reads need no checks
                // and go out together; a lane outside the event's reach multiplies by a zero
                // sample instead (not by a zero tap: the sample may be infinite).  No branches.
                const int i0 = pos - lane;
                const float *tp = fL + i0;
                const float t0v = tp[0], t1v = tp[kWave], t2v = tp[2 * kWave];
                const float x0 = static_cast<unsigned>(i0) < static_cast<unsigned>(F) ? xv : 0.0f;
                const float x1 = static_cast<unsigned>(i0 + kWave) < static_cast<unsigned>(F) ? xv : 0.0f;
                const float x2 = static_cast<unsigned>(i0 + 2 * kWave) < static_cast<unsigned>(F) ? xv : 0.0f;
                acc[b] = __builtin_fmaf(x0, t0v, acc[b]);
                if (b >= 1) acc[b >= 1 ? b - 1 : 0] = __builtin_fmaf(x1, t1v, acc[b >= 1 ? b - 1 : 0]);
                if (b >= 2) acc[b >= 2 ? b - 2 : 0] = __builtin_fmaf(x2, t2v, acc[b >= 2 ? b - 2 : 0]);
            }
        }
#pragma unroll
        for (int k = 0; k < kSparseBlocks; ++k) {
            if (k >= nPass) break;
            const int m = k * kWave + lane;
            const int time = CAUSAL ? (tHi - m) : (t0 + m);
            // the blocks of 64 outputs of a row complete each other's memory lines: keep them cached
            buffer_store<0>(bufOut, masked_offset(m < ttp && time >= t0 && time < t0 + tt, (r * T + time) * 4), 0,
                            acc[k] * Ts);
        }
    }
}

// VEC: rows are whole 16-byte vectors (T % 4 == 0, pointers 16-byte aligned)
// GATED: the staged samples are in * pdf(gate.u), computed once per staged sample
// DM: 0 = dense tiles run the register-window chains; 4..9 = dense tiles run on the matrix cores with a window
//     of DM blocks of 16 samples (VEC, U = 16, R = 16 rows, LD >= tile + 16 (DM - 1))
template <bool CAUSAL, bool VEC, int U, bool GATED, int DM>
__global__ __launch_bounds__(256, DM > 0 ? 2 : 1) void fir_tiled_kernel(float *__restrict__ out,
                                                        const float *__restrict__ in,
                                                        const float *__restrict__ filt,
                                                        int64_t rows, int T, int F, int TT, int LD, int R,
                                                        float Ts, FirGate gate)
{
    extern __shared__ __align__(16) float X[];
    // filter copy for the sparse path: taps -63 .. 191, zeros outside [0, F)
    float *fL = X + R * LD + (kWave - 1);
    uint32_t *nzCount = reinterpret_cast<uint32_t *>(X + R * LD + 4 * kWave);  // non-zero input samples and vectors, per wavefront
    uint32_t nonZero = 0;                                          // wave-uniform

    const int tid = threadIdx.x;
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), rows - row0));
    const int t0 = blockIdx.y * TT;                   // first output time of the tile
    const int tt = min(TT, T - t0);                   // outputs in this tile
    const int ttp = (tt + U - 1) & ~(U - 1);  // rounded up to whole chunks
    const int tHi = t0 + ttp - 1;                     // time stored at X[.][0] when reversed
    const int LD4 = LD >> 2;

    // The tile's rows as 32-bit offsets from its first row (a tile spans far less than 2 GiB).
    const BufferRsrc bufIn = make_buffer(in + row0 * static_cast<int64_t>(T));
    const BufferRsrc bufOut = make_buffer(out + row0 * static_cast<int64_t>(T));
    const BufferRsrc bufGate = make_buffer((GATED ? gate.u : in) + row0 * static_cast<int64_t>(T));
    auto gated = [&](float x, float u) { return x * spike_pdf(u, gate.theta, gate.tau, gate.gain); };

    // ---- stage: X[r][j] = in[row0+r][time(j)], zero outside the row;
    //      time(j) = t0 + j (correlation) or tHi - j (convolution)
    if (VEC) {
        // samples of the row that the tile needs: times [tA, tB), whole 16-byte vectors
        const int tA = CAUSAL ? max(0, tHi + 1 - LD) : t0;
        const int tB = CAUSAL ? min(T, tHi + 1) : min(T, t0 + LD);
        const int nq = (tB - tA) >> 2;               // source vectors per row
        const int jA = CAUSAL ? (tHi + 1 - tB) : 0;  // X columns [jA, jA + 4 nq) receive them
        {
            // vector g of the tile is vector g % nq of row g / nq; a lane's vectors are 256 apart, so its source and
            // destination offsets move by a fixed step plus a correction whenever the column wraps into the next row
            int r, col;
            divmod_small(tid, nq, 1.0f / static_cast<float>(nq), r, col);
            const int dr = 256 / nq, dc = 256 % nq;
            const int total = nRows * nq;
            int src = (r * T + tA + (col << 2)) * 4;
            int dst = (r * LD + (CAUSAL ? jA + ((nq - 1 - col) << 2) : (col << 2))) * 4;
            const int srcStep = (dr * T + dc * 4) * 4, srcWrap = srcStep + (T - nq * 4) * 4;
            const int dstStep = (dr * LD + (CAUSAL ? -dc : dc) * 4) * 4, dstWrap = dstStep + (LD + (CAUSAL ? nq : -nq) * 4) * 4;
            for (int g = tid; g < total; g += 256) {
                float4 v = buffer_load4(bufIn, src, 0);
                if (GATED) {
                    const float4 g = buffer_load4(bufGate, src, 0);
                    v = make_float4(gated(v.x, g.x), gated(v.y, g.y), gated(v.z, g.z), gated(v.w, g.w));
                }
                nonZero += count_nonzero(v);
                // (convolution: descending time, the vector lands mirrored)
                *reinterpret_cast<float4 *>(reinterpret_cast<char *>(X) + dst) = CAUSAL ? make_float4(v.w, v.z, v.y, v.x) : v;
                col += dc;
                const bool wrap = col >= nq;
                if (wrap) col -= nq;
                src += wrap ? srcWrap : srcStep;
                dst += wrap ? dstWrap : dstStep;
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
            const float *gsrc = (GATED ? gate.u : in) + (row0 + r) * static_cast<int64_t>(T);
            auto at = [&](int t) { return GATED ? gated(src[t], gsrc[t]) : src[t]; };
            const int j = j4 << 2;
            float4 v = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            const int tl = CAUSAL ? tHi - j - 3 : t0 + j;  // lowest time of the quad (X order is descending for conv)
            if (CAUSAL) {
                if (tl + 3 >= 0 && tl + 3 < T) v.x = at(tl + 3);
                if (tl + 2 >= 0 && tl + 2 < T) v.y = at(tl + 2);
                if (tl + 1 >= 0 && tl + 1 < T) v.z = at(tl + 1);
                if (tl >= 0 && tl < T) v.w = at(tl);
            } else {
                if (tl < T) v.x = at(tl);
                if (tl + 1 < T) v.y = at(tl + 1);
                if (tl + 2 < T) v.z = at(tl + 2);
                if (tl + 3 < T) v.w = at(tl + 3);
            }
            *reinterpret_cast<float4 *>(X + r * LD + j) = v;
            nonZero += count_nonzero(v);
        }
    }
    {
        const int i = tid - (kWave - 1);  // 256 lanes, taps -63 .. 192
        if (i < 3 * kWave) fL[i] = (i >= 0 && i < F) ? filt[i] : 0.0f;
    }
    if ((tid & (kWave - 1)) == 0) nzCount[tid / kWave] = nonZero;
    __syncthreads();

    // ---- sparse input: event-driven path
    {
        const uint32_t nz = nzCount[0] + nzCount[1] + nzCount[2] + nzCount[3];
        const uint32_t events = nz & 0xffffu, vectors = nz >> 16;
        const uint32_t samples = static_cast<uint32_t>(nRows) * static_cast<uint32_t>(LD);
        // The event-driven path pays per event: up to one event per 20 staged samples next to the matrix cores, one
        // per 32 next to the chains.  Spike trains that come in bursts (pooled ones: more than 3 events per 2
        // non-zero vectors) put most of a tile's events into a few rows, and the tile lasts as long as the wavefront
        // with the busiest rows: half that density for them.
        constexpr uint32_t kPer = DM > 0 ? 20u : 32u;
        const uint32_t per = 2u * events > 3u * vectors ? 2u * kPer : kPer;
        if (F <= kSparseMaxTaps && LD <= kSparseBlocks * kWave && events * per <= samples) {
            fir_sparse_tile<CAUSAL>(bufOut, X, fL, nRows, LD, ttp, t0, tt, tHi, T, F, Ts);
            return;
        }
    }

    // ---- dense input on the matrix cores.  The tile's rows are cut into blocks of 16 outputs; the blocks of all rows
    // are the "columns", and a wavefront takes 16 consecutive columns at a time.  The 16 outputs of a column are the
    // product of a banded Toeplitz matrix of the filter with the DM blocks of X that start where the column does:
    //     Y[16b + i] = sum_{d < DM} sum_{kk < 16} filt[16d + kk - i] * X[16(b + d) + kk].
    // v_mfma_f32_16x16x4_f32 takes 4 of the 16 kk per instruction: lane (c = lane % 16, h = lane / 16) supplies
    // X[16(b + d) + 4h + v] of column c for instruction v = 0..3 - one 16-byte LDS read per d, 64 d bytes on from
    // the first, an offset that sits in the instruction - and filt[16d + 4h + v - i] for i = lane % 16 (from the
    // zero-padded filter copy, kept in 4 DM registers); its accumulator holds outputs 4h..4h+3 of column c, which
    // it stores straight to memory.  The rows' zero padding in LDS ends every window where its row ends.  The
    // matrix instruction adds 4 products per step in its own order: results agree with the chain to rounding,
    // not bit for bit.  A structural zero times a non-finite sample would be NaN where the chain has no such
    // term: columns whose results contain a NaN are computed again as sequential chains.
    if constexpr (DM > 0) {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const int lane = tid & (kWave - 1), wave = tid / kWave;
        const int c = lane & 15, h = lane >> 4;
        float a[DM][4];
        {
            const float *fa = fL + (4 * h - c);
#pragma unroll
            for (int d = 0; d < DM; ++d)
#pragma unroll
                for (int v = 0; v < 4; ++v) a[d][v] = fa[16 * d + v];
        }
        const int nb = ttp >> 4;  // columns per row
        const int cols = nRows * nb;
        // (a wavefront's columns beyond the last row fall into rows of LDS that were not staged: their results
        // are not stored)
        RowCol rb;
        rb.init(16 * wave + c, nb, 1.0f / static_cast<float>(nb));
        const int stepR = 64 / nb, stepB = 64 % nb;
        for (int g0 = 16 * wave; g0 < cols; g0 += 64, rb.advance(stepR, stepB, nb)) {
            const bool on = g0 + c < cols;
            const int r = rb.r, b = rb.c;
            const int m0 = 16 * b + 4 * h;
            const float *xp = X + r * LD + m0;
            float4 w[DM];
#pragma unroll
            for (int d = 0; d < DM; ++d) w[d] = *reinterpret_cast<const float4 *>(xp + 16 * d);
            f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int d = 0; d < DM; ++d) {
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][0], w[d].x, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][1], w[d].y, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][2], w[d].z, acc, 0, 0, 0);
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][3], w[d].w, acc, 0, 0, 0);
            }
            // (only in columns that are part of the tile: the others hold whatever LDS held)
            const bool nan = on & (__builtin_isunordered(acc.x, acc.y) | __builtin_isunordered(acc.z, acc.w));
            if (__builtin_amdgcn_ballot_w64(nan) != 0) {
                float y[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    float sum = 0.0f;
                    for (int i = 0; i < F; ++i) sum = __builtin_fmaf(xp[j + i], fL[i], sum);
                    y[j] = sum;
                }
                acc = f32x4{y[0], y[1], y[2], y[3]};
            }
            // times t0 + m0 .. (correlation) or tHi - m0 - 3 .. tHi - m0 (convolution); both are multiples of 4 and so
            // is the tile's end, so the vector is all in or all out
            const int tl = CAUSAL ? (tHi - m0 - 3) : (t0 + m0);
            const bool valid = on && tl >= t0 && tl + 3 < t0 + tt;
            const float4 y = CAUSAL ? make_float4(acc.w * Ts, acc.z * Ts, acc.y * Ts, acc.x * Ts)
                                    : make_float4(acc.x * Ts, acc.y * Ts, acc.z * Ts, acc.w * Ts);
            // the columns of a wavefront are consecutive in memory: neighbouring stores complete each other's lines
            buffer_store4<0>(bufOut, masked_offset(valid, (r * T + tl) * 4), 0, y);
        }
        return;
    }

    // ---- compute: work item = (row, chunk of 8 outputs), row-major over lanes
    const int nChunks = ttp / U;
    const int items = nRows * nChunks;
    const int F4 = F & ~3;
    RowCol item;
    item.init(tid, nChunks, 1.0f / static_cast<float>(nChunks));
    const int itemDr = 256 / nChunks, itemDc = 256 % nChunks;

    for (int w = tid; w < items; w += 256, item.advance(itemDr, itemDc, nChunks)) {
        const int r = item.r;
        const int m0 = item.c * U;
        float acc[U];
#pragma unroll
        for (int j = 0; j < U; ++j) acc[j] = 0.0f;

        constexpr int NQ = U / 4 + 1;
        const float4 *xq = reinterpret_cast<const float4 *>(X + r * LD + m0);
        float4 q[NQ];
#pragma unroll
        for (int v = 0; v < NQ; ++v) q[v] = xq[v];
        int i = 0, qi = NQ;
        for (; i + 4 * NQ <= F4; i += 4 * NQ, qi += NQ) TripBlocks<U, 0>::run(acc, q, xq, qi, filt + i);
        TailBlocks<U, 0>::run(acc, q, xq, qi, filt + i, F - i);

        // ---- store the U outputs: times t0+m0 .. (correlation) or tHi-m0-(U-1) .. tHi-m0 (convolution)
        float y[U];
#pragma unroll
        for (int j = 0; j < U; ++j) y[j] = (CAUSAL ? acc[U - 1 - j] : acc[j]) * Ts;
        const int tl = CAUSAL ? (tHi - m0 - (U - 1)) : (t0 + m0);  // lowest time of the chunk
        if (VEC) {
            // tl is a multiple of 4 and so is the tile's end, so each vector is all in or all out.
            // The vectors of one lane complete each other's memory lines: keep them cached.
            const int off = (r * T + tl) * 4;
#pragma unroll
            for (int v = 0; v < U / 4; ++v)
                if (tl + 4 * v >= t0 && tl + 4 * v + 3 < t0 + tt)
                    buffer_store4<0>(bufOut, off + 16 * v, 0, make_float4(y[4 * v], y[4 * v + 1], y[4 * v + 2], y[4 * v + 3]));
        } else {
            float *dst = out + (row0 + r) * static_cast<int64_t>(T);
#pragma unroll
            for (int v = 0; v < U / 4; ++v) {
                const int tv = tl + 4 * v;
                if (tv >= t0 && tv + 3 < t0 + tt) {
                    const float4u q = {y[4 * v], y[4 * v + 1], y[4 * v + 2], y[4 * v + 3]};
                    *reinterpret_cast<float4u *>(dst + tv) = q;   // 16 bytes at any alignment
                } else {
#pragma unroll
                    for (int j = 4 * v; j < 4 * v + 4; ++j)
                        if (tl + j >= t0 && tl + j < t0 + tt) dst[tl + j] = y[j];
                }
            }
        }
    }
}

struct FirPlan {
    int U, TT, LD, R, nTiles;
};

// Chooses outputs per lane, the time tile, the LDS row pitch and the rows per work-group.
static bool plan_fir(int64_t rows, int64_t T, int64_t F, FirPlan &best)
{
    if (F < 1 || T > kBufferMaxT) return false;
    double bestScore = -1.0;
    for (int U = 16; U >= 8; U -= 8) {
        // a row of X holds ttp + F + 4 samples (chunk-rounded tile, halo, window over-read)
        const int64_t ttMax = (kFirMaxPitch - 4 - F) & ~static_cast<int64_t>(U - 1);
        if (ttMax < 64) continue;
        const int64_t nTiles = ceil_div(T, ttMax);
        if (nTiles > 65535) continue;
        int64_t TT = ceil_div(ceil_div(T, nTiles), U) * U;
        if (nTiles == 1) TT = T;
        const int64_t ttp = ceil_div(TT, U) * U;
        const int64_t LD = (ttp + F + 4 + 3) & ~static_cast<int64_t>(3);
        const int64_t nChunks = ttp / U;
        const int64_t rMax = kFirMaxLdsFloats / LD;
        if (rMax < 1) continue;
        // per-item work: F taps on U outputs plus a fixed prologue/epilogue; rows per group: fill
        // the 256 lanes evenly with (row, chunk) items and prefer small tiles (more groups per CU
        // overlap staging with compute)
        const double perOutput = (static_cast<double>(F) + 60.0 / U) * static_cast<double>(ttp) /
                                 static_cast<double>(TT < T ? TT : T);
        for (int64_t r = 1; r <= rMax && r <= 64; ++r) {
            const int64_t items = r * nChunks;
            const double eff = static_cast<double>(items) / static_cast<double>(ceil_div(items, 256) * 256);
            const double score = eff / perOutput - (items < 256 ? 0.25 / F : 0.0) -
                                 0.25 / F * static_cast<double>(r * LD) / kFirMaxLdsFloats;
            if (score > bestScore) {
                bestScore = score;
                best.U = U;
                best.TT = static_cast<int>(TT);
                best.LD = static_cast<int>(LD);
                best.R = static_cast<int>(r);
                best.nTiles = static_cast<int>(nTiles);
            }
        }
    }
    if (bestScore < 0.0) return false;
    if (best.R > rows) best.R = static_cast<int>(rows);
    return true;
}

// The plan of the matrix-core variant: tiles of 16 rows, whole blocks of 16 outputs, and a row pitch that holds
// the window of the tile's last block.
static bool plan_fir_mfma(int64_t rows, int64_t T, int64_t F, FirPlan &best)
{
    if (F < kFirMfmaMinTaps || F > kFirMfmaMaxTaps || T > kBufferMaxT || T < 16) return false;
    const int64_t D = (F + 14) / 16 + 1;
    const int64_t halo = (F + 4 > 16 * (D - 1) ? F + 4 : 16 * (D - 1));
    const int64_t ttMax = (kFirMaxPitch - 4 - halo) & ~static_cast<int64_t>(15);
    if (ttMax < 64) return false;
    const int64_t nTiles = ceil_div(T, ttMax);
    if (nTiles > 65535) return false;
    int64_t TT = ceil_div(ceil_div(T, nTiles), 16) * 16;
    if (nTiles == 1) TT = T;
    const int64_t ttp = ceil_div(TT, 16) * 16;
    best.U = 16;
    best.TT = static_cast<int>(TT);
    best.LD = static_cast<int>((ttp + halo + 3) & ~static_cast<int64_t>(3));
    best.R = 16;
    best.nTiles = static_cast<int>(nTiles);
    return true;
}

template <bool CAUSAL, bool VEC, int U, bool GATED, int DM = 0>
static void launch_tiled(const FirPlan &p, float *out, const float *in, const float *filt, int64_t rows, int64_t T,
                         int64_t F, float Ts, const FirGate &gate, hipStream_t stream)
{
    dim3 grid(static_cast<unsigned>(ceil_div(rows, p.R)), static_cast<unsigned>(p.nTiles)), block(256);
    // rows, the zero-padded filter copy of the sparse path (256 floats) and four counters
    const size_t lds = (static_cast<size_t>(p.R) * p.LD + 4 * kWave + 4) * sizeof(float);
    hipLaunchKernelGGL((fir_tiled_kernel<CAUSAL, VEC, U, GATED, DM>), grid, block, lds, stream, out, in, filt, rows,
                       static_cast<int>(T), static_cast<int>(F), p.TT, p.LD, p.R, Ts, gate);
}

template <bool CAUSAL, bool GATED>
static int launch_fir(float *out, const float *in, const float *filt, int64_t rows, int64_t T,
                      int64_t F, float Ts, const FirGate &gate, hipStream_t stream)
{
    if (rows < 0 || T < 0 || F < 0) return SLAYER_EINVAL;
    if (rows == 0 || T == 0) return SLAYER_OK;
    if (!out || !in || (F > 0 && !filt) || (GATED && !gate.u)) return SLAYER_EINVAL;
    if (T >= (1LL << 30)) return SLAYER_EUNSUPPORTED;

    const bool vec = (T % 4 == 0) && aligned16(out) && aligned16(in) && (!GATED || aligned16(gate.u));
    // The correlation's input is a gradient, i.e. dense: from 34 taps on, where the chain kernels are bound by
    // FMA issue, it runs on the matrix cores (the gated one too when its rows fit that kernel's linear layout).
    // The convolution does not: its input is mostly spike trains, which the tiled kernel's event-driven path
    // serves at the speed of a copy and with the bits of the chain.
    if (!CAUSAL && !generic_forced() && launch_fir_corr_mfma(out, in, filt, rows, T, F, Ts, gate, stream))
        return launch_status();
    {
    FirPlan p;
    // Longer filters on rows of whole vectors: the tiled kernel whose dense tiles run on the matrix cores (its
    // sparse tiles, spike trains, keep the event-driven path and the bits of the chain).
    if (!generic_forced() && vec && plan_fir_mfma(rows, T, F, p) && ceil_div(rows, p.R) < (1LL << 31)) {
        switch ((F + 14) / 16 + 1) {
            case 4: launch_tiled<CAUSAL, true, 16, GATED, 4>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
            case 5: launch_tiled<CAUSAL, true, 16, GATED, 5>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
            case 6: launch_tiled<CAUSAL, true, 16, GATED, 6>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
            case 7: launch_tiled<CAUSAL, true, 16, GATED, 7>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
            case 8: launch_tiled<CAUSAL, true, 16, GATED, 8>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
            default: launch_tiled<CAUSAL, true, 16, GATED, 9>(p, out, in, filt, rows, T, F, Ts, gate, stream); break;
        }
        return launch_status();
    }
    }
    // Register-only kernel for short filters (the op is then a stream).
    const int64_t directMax = 33;
    // (not with a gate: every lane would evaluate the gate for its whole window).
    if (!GATED && !generic_forced() && vec && F >= 1 && F <= directMax && T < (1LL << 28) && rows * (T / 4) < (1LL << 32)) {
        const int U = F <= 17 ? 4 : 8;
        const int64_t chunksPerRow = ceil_div(T / 4, U / 4);
        const int64_t chunks = rows * chunksPerRow;
        const dim3 grid(static_cast<unsigned>(ceil_div(chunks, 256)));
        const FastDiv byRow = make_fastdiv(static_cast<uint32_t>(chunksPerRow));
#define SLAYER_FIR_DIRECT(NV, UU)                                                                                  \
    hipLaunchKernelGGL((fir_direct_kernel<CAUSAL, NV, UU>), grid, dim3(256), 0, stream, out, in, filt,             \
                       static_cast<uint32_t>(chunks), static_cast<int>(T), static_cast<int>(F), byRow, Ts)
        if (F <= 5) SLAYER_FIR_DIRECT(2, 4);
        else if (F <= 9) SLAYER_FIR_DIRECT(3, 4);
        else if (F <= 13) SLAYER_FIR_DIRECT(4, 4);
        else if (F <= 17) SLAYER_FIR_DIRECT(5, 4);
        else if (F <= 25) SLAYER_FIR_DIRECT(8, 8);
        else SLAYER_FIR_DIRECT(10, 8);
#undef SLAYER_FIR_DIRECT
        return launch_status();
    }
    FirPlan p;
    if (!generic_forced() && plan_fir(rows, T, F, p) && ceil_div(rows, p.R) < (1LL << 31)) {
        if (vec && p.U == 16) launch_tiled<CAUSAL, true, 16, GATED>(p, out, in, filt, rows, T, F, Ts, gate, stream);
        else if (vec) launch_tiled<CAUSAL, true, 8, GATED>(p, out, in, filt, rows, T, F, Ts, gate, stream);
        else if (p.U == 16) launch_tiled<CAUSAL, false, 16, GATED>(p, out, in, filt, rows, T, F, Ts, gate, stream);
        else launch_tiled<CAUSAL, false, 8, GATED>(p, out, in, filt, rows, T, F, Ts, gate, stream);
        return launch_status();
    }
    const int64_t tBlocks = ceil_div(T, 256);
    if (tBlocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    dim3 grid(static_cast<unsigned>(tBlocks), static_cast<unsigned>(rows < 65535 ? rows : 65535));
    hipLaunchKernelGGL((fir_generic_kernel<CAUSAL, GATED>), grid, dim3(256), 0, stream, out, in, filt, rows, T,
                       F, Ts, gate);
    return launch_status();
}

}  // namespace slayer

extern "C" int slayer_conv_f32(float *out, const float *in, const float *filt, int64_t nNeurons,
                               int64_t T, int64_t F, float Ts, void *stream)
{
    return slayer::launch_fir<true, false>(out, in, filt, nNeurons, T, F, Ts, slayer::FirGate{nullptr, 0.0f, 1.0f, 0.0f},
                                           static_cast<hipStream_t>(stream));
}

extern "C" int slayer_corr_f32(float *out, const float *in, const float *filt, int64_t nNeurons,
                               int64_t T, int64_t F, float Ts, void *stream)
{
    return slayer::launch_fir<false, false>(out, in, filt, nNeurons, T, F, Ts, slayer::FirGate{nullptr, 0.0f, 1.0f, 0.0f},
                                            static_cast<hipStream_t>(stream));
}

extern "C" int slayer_spike_bwd_corr_f32(float *gradIn, const float *gradOut, const float *u, const float *filt,
                                         int64_t nNeurons, int64_t T, int64_t F, float theta, float tau,
                                         float scale, float Ts, void *stream)
{
    if (tau == 0.0f) return SLAYER_EINVAL;
    return slayer::launch_fir<false, true>(gradIn, gradOut, filt, nNeurons, T, F, Ts,
                                           slayer::FirGate{u, theta, tau, scale / tau},
                                           static_cast<hipStream_t>(stream));
}

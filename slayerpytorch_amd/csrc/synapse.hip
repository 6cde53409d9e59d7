// Per-timestep synapses on [N][C][H][W][T] tensors (time innermost): 2-D cross-correlation over
// (H, W) applied to every time sample, and its two gradients.  The reference's layers obtain this
// from conv3d / conv_transpose3d with a kernel of time extent 1 (src/slayer.py:499-507 conv,
// :565-575 pool, :631-643 convTranspose, :732-748 unpool).
//
// With time innermost the filter does not depend on the fastest axis, so every lane owns a run of
// consecutive time samples (one 16-byte vector) of one pixel: loads and stores are contiguous along
// T for any stride, padding or dilation, and the weights are wave-uniform.  Forward and input
// gradient are one gather: on the matrix cores for layers with at least 16 destination channels
// and source channels that fill passes of about 144 taps (a source patch in LDS, the taps as the
// reduction axis), on the vector ALUs otherwise (a general kernel, and one that keeps the columns
// of a filter row in registers for layers with one or two destination channels).  The weight
// gradient, a matrix product with time as the reduction axis, runs on the matrix cores from a
// source patch in LDS (from global memory for patches that do not fit, and a vector kernel for
// small or unaligned shapes); pooling has a streaming input gradient.  The forward gather and the
// weight gradient multiply with bf16 matrix instructions over operands split into three bf16 parts
// (fir_core.h); the input gradient, whose source is a gradient tensor, with the fp32 instruction.
// Work-groups that read the same rows are kept on the same die (xcd_contiguous).
#include <atomic>
#include <type_traits>

#include "common.h"
#include "fir_core.h"   // split_bf16, mfma_bf16

namespace slayer {

struct SynGeom {
    int N, C, H, W, T, O, KH, KW, sH, sW, pH, pW, dH, dW, groups, OH, OW;
};

// ---- gather kernel: forward and input gradient --------------------------------------------------
// dst[n][m][a][b][t] = sum over the source channels q of m's group and the taps (i, j) of
//     weight(m, q, i, j) * src[n][q][ya][xb][t]
// forward  (BACKWARD = false): dst = out, src = in,      ya = a*sH - pH + i*dH
// gradient (BACKWARD = true):  dst = gradIn, src = gradOut, ya = (a + pH - i*dH) / sH where that
//                              division is exact (the output rows whose tap i read input row a)
// A lane owns VEC consecutive time samples of one destination pixel and MB destination channels
// (accumulators in registers); a work-group of 256 lanes covers 256 consecutive vectors of the
// (a, b, t) volume, which is also their order in memory, so stores are one contiguous run per
// channel.  The work-group's MB x K weights sit in LDS, tap-major, and are read as broadcasts.
struct GatherArgs {
    const float *src;
    float *dst;
    const float *w;
    int SC, SH, SW, DC, DH, DW, T;
    int Qg, Mg, mBlocks, groups;  // source / destination channels per group, MB-blocks per group
    int KH, KW, Cg, Og;
    int mulH, mulW, offH, offW, stepH, stepW;  // source row numerator = a*mulH + offH + i*stepH
    FastDiv divH, divW;                        // ... divided by the stride in the gradient
    int P;                                     // vectors per destination channel plane = DH*DW*T/VEC
    int chunks;                                // work-groups per (n, group, m-block)
    FastDiv byChunks, byMBlocks, byGroups, byTV, byDW;
};

constexpr int kTapChunk = 256;  // taps of weights held in LDS at a time

template <int VEC> struct TimeVec;
template <> struct TimeVec<4> {
    float4 v;
    __device__ __forceinline__ void load(BufferRsrc b, int off, int uniform = 0) { v = buffer_load4<0>(b, off, uniform); }
    __device__ __forceinline__ void zero() { v = make_float4(0.f, 0.f, 0.f, 0.f); }
    __device__ __forceinline__ void fma(float w, const TimeVec &x)
    {
        v.x = fmaf(w, x.v.x, v.x);
        v.y = fmaf(w, x.v.y, v.y);
        v.z = fmaf(w, x.v.z, v.z);
        v.w = fmaf(w, x.v.w, v.w);
    }
    __device__ __forceinline__ void store(BufferRsrc b, int off) const { buffer_store4<kStream>(b, off, 0, v); }
    __device__ __forceinline__ float dot(const TimeVec &x, float acc) const
    {
        acc = fmaf(v.x, x.v.x, acc);
        acc = fmaf(v.y, x.v.y, acc);
        acc = fmaf(v.z, x.v.z, acc);
        return fmaf(v.w, x.v.w, acc);
    }
};
template <> struct TimeVec<1> {
    float v;
    __device__ __forceinline__ void load(BufferRsrc b, int off, int uniform = 0)
    {
        v = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(b, off, uniform, 0));
    }
    __device__ __forceinline__ void zero() { v = 0.f; }
    __device__ __forceinline__ void fma(float w, const TimeVec &x) { v = fmaf(w, x.v, v); }
    __device__ __forceinline__ void store(BufferRsrc b, int off) const { buffer_store<kStream>(b, off, 0, v); }
    __device__ __forceinline__ float dot(const TimeVec &x, float acc) const { return fmaf(v, x.v, acc); }
};

template <int MB, int VEC, bool BACKWARD, bool STRIDED>
__global__ __launch_bounds__(256) void synapse_gather_kernel(GatherArgs g)
{
    __shared__ __attribute__((aligned(16))) float wl[kTapChunk * MB];

    // work-group -> (batch item, group, block of MB destination channels, chunk of 256 vectors);
    // neighbouring chunks read overlapping source rows, so they are kept on one die
    // (the blocks of destination channels of one chunk read the same source rows: they are neighbours)
    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    const uint32_t nc = fastdiv(rest, g.byMBlocks);
    const int mb0 = static_cast<int>(rest - nc * g.byMBlocks.d) * MB;  // first channel of the block, within the group
    const uint32_t ng = fastdiv(nc, g.byChunks);
    const int chunk = static_cast<int>(nc - ng * g.byChunks.d);
    const uint32_t n = fastdiv(ng, g.byGroups);
    const int grp = static_cast<int>(ng - n * g.byGroups.d);

    const int p = chunk * 256 + static_cast<int>(threadIdx.x);
    const bool live = p < g.P;
    const uint32_t pix = fastdiv(static_cast<uint32_t>(live ? p : 0), g.byTV);
    const int tv = (live ? p : 0) - static_cast<int>(pix * g.byTV.d);
    const int a = static_cast<int>(fastdiv(pix, g.byDW));
    const int b = static_cast<int>(pix) - a * g.DW;

    const int64_t srcPlane = static_cast<int64_t>(g.SH) * g.SW * g.T;  // floats per source channel
    const BufferRsrc srcB = make_buffer(g.src + (static_cast<int64_t>(n) * g.SC + static_cast<int64_t>(grp) * g.Qg) * srcPlane);
    const int rowBytes = g.SW * g.T * 4, pixBytes = g.T * 4;
    const int planeBytes = static_cast<int>(srcPlane) * 4;
    const int laneBytes = tv * VEC * 4;
    const int yNum0 = a * g.mulH + g.offH, xNum0 = b * g.mulW + g.offW;
    // unstrided sources: position and byte offset of the lane before any tap offset, and a buffer
    // that starts at the smallest tap offset
    const int yBase = a * g.mulH, xBase = b * g.mulW;
    const int laneOff = yBase * rowBytes + xBase * pixBytes + laneBytes;
    const int minDy = g.offH + min(0, (g.KH - 1) * g.stepH), minDx = g.offW + min(0, (g.KW - 1) * g.stepW);
    const int minTapOff = minDy * rowBytes + minDx * pixBytes;
    const BufferRsrc srcT = make_buffer(reinterpret_cast<const char *>(
        g.src + (static_cast<int64_t>(n) * g.SC + static_cast<int64_t>(grp) * g.Qg) * srcPlane) + minTapOff);

    TimeVec<VEC> acc[MB];
#pragma unroll
    for (int m = 0; m < MB; ++m) acc[m].zero();

    const int KK = g.KH * g.KW;
    const int K = g.Qg * KK;
    for (int k0 = 0; k0 < K; k0 += kTapChunk) {
        const int kc = min(kTapChunk, K - k0);
        __syncthreads();
        for (int e = threadIdx.x; e < kc * MB; e += 256) {
            const int tap = k0 + e / MB, m = mb0 + e % MB;
            const int q = tap / KK, ij = tap - q * KK;
            float v = 0.f;
            if (m < g.Mg) {
                const int64_t idx = BACKWARD
                    ? (static_cast<int64_t>(grp * g.Og + q) * g.Cg + m) * KK + ij
                    : (static_cast<int64_t>(grp * g.Og + m) * g.Cg + q) * KK + ij;
                v = g.w[idx];
            }
            wl[e] = v;
        }
        __syncthreads();

        // taps k0 .. k0+kc in (q, i, j) order; the counters are wave-uniform.  The load of a tap is
        // issued one tap ahead of the multiply-adds that use it.
        int q = k0 / KK, ij = k0 - q * KK;
        int i = ij / g.KW, j = ij - i * g.KW;
        auto fetch = [&](bool inChunk) {
            const int dy = g.offH + i * g.stepH, dx = g.offW + j * g.stepW;  // wave-uniform
            TimeVec<VEC> x;
            if (MB < 4 && !STRIDED) {
                // few channels per lane: the loads dominate, and they measured faster with the whole
                // offset in the vector register (318 us against 272 us on 2 destination channels)
                const int y = yBase + dy, xx = xBase + dx;
                const bool ok = static_cast<unsigned>(y) < static_cast<unsigned>(g.SH) &&
                                static_cast<unsigned>(xx) < static_cast<unsigned>(g.SW);
                x.load(srcB, masked_offset(ok && live && inChunk, q * planeBytes + y * rowBytes + xx * pixBytes + laneBytes));
            } else if (STRIDED) {
                const int yNum = yNum0 + i * g.stepH, xNum = xNum0 + j * g.stepW;
                const uint32_t yq = fastdiv(static_cast<uint32_t>(yNum), g.divH);
                const uint32_t xq = fastdiv(static_cast<uint32_t>(xNum), g.divW);
                const bool ok = yNum >= 0 && xNum >= 0 && static_cast<int>(yq * g.divH.d) == yNum &&
                                static_cast<int>(xq * g.divW.d) == xNum && static_cast<int>(yq) < g.SH &&
                                static_cast<int>(xq) < g.SW;
                x.load(srcB, masked_offset(ok && live && inChunk, q * planeBytes + static_cast<int>(yq) * rowBytes +
                                                                      static_cast<int>(xq) * pixBytes + laneBytes));
            } else {
                // the lane's own offset does not change from tap to tap; the tap's offset is uniform and
                // travels in a scalar register (counted from the smallest tap offset, so never negative)
                const bool ok = static_cast<unsigned>(yBase + dy) < static_cast<unsigned>(g.SH) &&
                                static_cast<unsigned>(xBase + dx) < static_cast<unsigned>(g.SW);
                x.load(srcT, masked_offset(ok && live && inChunk, laneOff),
                       q * planeBytes + dy * rowBytes + dx * pixBytes - minTapOff);
            }
            if (++j == g.KW) {
                j = 0;
                if (++i == g.KH) { i = 0; ++q; }
            }
            return x;
        };
        auto madd = [&](const TimeVec<VEC> &x, int t) {
            const float *wt = wl + t * MB;
            if constexpr (MB >= 4) {
#pragma unroll
                for (int m = 0; m < MB; m += 4) {
                    const float4 w4 = *reinterpret_cast<const float4 *>(wt + m);
                    acc[m].fma(w4.x, x);
                    acc[m + 1].fma(w4.y, x);
                    acc[m + 2].fma(w4.z, x);
                    acc[m + 3].fma(w4.w, x);
                }
            } else {
#pragma unroll
                for (int m = 0; m < MB; ++m) acc[m].fma(wt[m], x);
            }
        };
        // two taps per trip, so that the two operand registers swap roles without being copied
        TimeVec<VEC> xa = fetch(true);
        for (int t = 0; t < kc; t += 2) {
            const TimeVec<VEC> xb = fetch(t + 1 < kc);
            madd(xa, t);
            xa = fetch(t + 2 < kc);
            if (t + 1 < kc) madd(xb, t + 1);
        }
    }

    const int64_t dstPlane = static_cast<int64_t>(g.DH) * g.DW * g.T;
    const BufferRsrc dstB = make_buffer(g.dst + (static_cast<int64_t>(n) * g.DC + static_cast<int64_t>(grp) * g.Mg) * dstPlane);
    const int dstPlaneBytes = static_cast<int>(dstPlane) * 4;
#pragma unroll
    for (int m = 0; m < MB; ++m)
        acc[m].store(dstB, masked_offset(live && mb0 + m < g.Mg, (mb0 + m) * dstPlaneBytes + p * VEC * 4));
}


// ---- gather with few destination channels: several pixels of a row per lane ---------------------------
// With one or two destination channels (the input gradient of a network's first layer) the kernel above
// issues one 16-byte load per 4 or 8 multiply-adds and is bound by its loads.  Here a lane owns PX adjacent
// destination pixels of one row (unit stride and dilation along W: pixel p's tap j reads source column
// p + j or p - j, so the PX pixels' KW taps fall on E = PX + KW - 1 distinct columns): per source channel and
// filter row it loads those columns once, and each loaded vector feeds every (pixel, tap) pair that
// lands on it - PX * KW * MB * 4 multiply-adds per E loads.  KW is a template parameter, so which pairs those
// are is known at compile time and the filter row's weights sit in registers; the E loads of a filter row are
// issued one row ahead of its multiply-adds (two rows per trip, so that the two sets of registers swap roles
// without copies).  Weights come from LDS in chunks of whole filter rows, [row][j][m].
constexpr int kGatherRowPx = 4;

template <int MB, int KW, bool BACKWARD>
__global__ __launch_bounds__(256) void synapse_gather_row_kernel(GatherArgs g)
{
    constexpr int PX = kGatherRowPx, E = PX + KW - 1;
    constexpr int kRows = kTapChunk / KW;                 // filter rows per chunk of weights
    __shared__ __attribute__((aligned(16))) float wl[kRows * KW * MB];

    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    const uint32_t nc = fastdiv(rest, g.byMBlocks);
    const int mb0 = static_cast<int>(rest - nc * g.byMBlocks.d) * MB;
    const uint32_t ng = fastdiv(nc, g.byChunks);
    const int chunk = static_cast<int>(nc - ng * g.byChunks.d);
    const uint32_t n = fastdiv(ng, g.byGroups);
    const int grp = static_cast<int>(ng - n * g.byGroups.d);

    // lane -> (row a, group of PX pixels, vector of time samples); g.P counts those, g.byDW divides by the
    // pixel groups per row
    const int p = chunk * 256 + static_cast<int>(threadIdx.x);
    const bool live = p < g.P;
    const uint32_t pg = fastdiv(static_cast<uint32_t>(live ? p : 0), g.byTV);
    const int tv = (live ? p : 0) - static_cast<int>(pg * g.byTV.d);
    const int a = static_cast<int>(fastdiv(pg, g.byDW));
    const int b0 = (static_cast<int>(pg) - a * static_cast<int>(g.byDW.d)) * PX;

    const int64_t srcPlane = static_cast<int64_t>(g.SH) * g.SW * g.T;
    const BufferRsrc srcB = make_buffer(g.src + (static_cast<int64_t>(n) * g.SC + static_cast<int64_t>(grp) * g.Qg) * srcPlane);
    const int rowBytes = g.SW * g.T * 4, pixBytes = g.T * 4, planeBytes = static_cast<int>(srcPlane) * 4;
    const int yBase = a * g.mulH;
    // source column of pixel p, tap j: b0 + p + offW + j * stepW with stepW = 1 (forward) or -1 (gradient), i.e.
    // x0 + e with e = p + j or p - j + KW - 1, 0 <= e < E
    const int x0 = b0 + g.offW - (BACKWARD ? KW - 1 : 0);
    // the lane's columns: byte offsets within a source row, masked where the column is outside the image
    int colOff[E];
#pragma unroll
    for (int e = 0; e < E; ++e)
        colOff[e] = masked_offset(live && static_cast<unsigned>(x0 + e) < static_cast<unsigned>(g.SW), (x0 + e) * pixBytes + tv * 16);

    TimeVec<4> acc[PX][MB];
#pragma unroll
    for (int px = 0; px < PX; ++px)
#pragma unroll
        for (int m = 0; m < MB; ++m) acc[px][m].zero();

    const int KK = g.KH * KW;
    const int rows = g.Qg * g.KH;                      // (source channel, filter row) pairs
    for (int r0 = 0; r0 < rows; r0 += kRows) {
        const int rc = min(kRows, rows - r0);
        __syncthreads();
        for (int e = threadIdx.x; e < rc * KW * MB; e += 256) {
            const int tap = r0 * KW + e / MB, m = mb0 + e % MB;   // tap in (q, i, j) order
            const int q = tap / KK, ij = tap - q * KK;
            float v = 0.f;
            if (m < g.Mg) {
                const int64_t idx = BACKWARD
                    ? (static_cast<int64_t>(grp * g.Og + q) * g.Cg + m) * KK + ij
                    : (static_cast<int64_t>(grp * g.Og + m) * g.Cg + q) * KK + ij;
                v = g.w[idx];
            }
            wl[e] = v;
        }
        __syncthreads();

        int q = r0 / g.KH, i = r0 - q * g.KH;          // the filter row to load next (wave-uniform)
        auto fetch = [&](TimeVec<4> (&X)[E], bool more) {
            const int y = yBase + g.offH + i * g.stepH;
            const bool ok = more && static_cast<unsigned>(y) < static_cast<unsigned>(g.SH);
            const int rowOff = q * planeBytes + y * rowBytes;
#pragma unroll
            for (int e = 0; e < E; ++e) X[e].load(srcB, ok && colOff[e] != kOutOfRange ? colOff[e] + rowOff : kOutOfRange);
            if (++i == g.KH) { i = 0; ++q; }
        };
        auto madd = [&](const TimeVec<4> (&X)[E], int row) {
            float w[KW][MB];
            const float *wr = wl + row * KW * MB;
#pragma unroll
            for (int j = 0; j < KW; ++j)
#pragma unroll
                for (int m = 0; m < MB; ++m) w[j][m] = wr[j * MB + m];
#pragma unroll
            for (int e = 0; e < E; ++e)
#pragma unroll
                for (int px = 0; px < PX; ++px) {
                    const int j = BACKWARD ? px - e + KW - 1 : e - px;
                    if (j >= 0 && j < KW) {
#pragma unroll
                        for (int m = 0; m < MB; ++m) acc[px][m].fma(w[j][m], X[e]);
                    }
                }
        };
        TimeVec<4> XA[E], XB[E];
        fetch(XA, true);
        for (int r = 0; r < rc; r += 2) {
            fetch(XB, r + 1 < rc);
            madd(XA, r);
            fetch(XA, r + 2 < rc);
            if (r + 1 < rc) madd(XB, r + 1);
        }
    }

    const int64_t dstPlane = static_cast<int64_t>(g.DH) * g.DW * g.T;
    const BufferRsrc dstB = make_buffer(g.dst + (static_cast<int64_t>(n) * g.DC + static_cast<int64_t>(grp) * g.Mg) * dstPlane);
    const int dstPlaneBytes = static_cast<int>(dstPlane) * 4;
#pragma unroll
    for (int px = 0; px < PX; ++px)
#pragma unroll
        for (int m = 0; m < MB; ++m)
            acc[px][m].store(dstB, masked_offset(live && b0 + px < g.DW && mb0 + m < g.Mg,
                                                 (mb0 + m) * dstPlaneBytes + ((a * g.DW + b0 + px) * g.T) * 4 + tv * 16));
}


// Input gradient of a one-channel synapse whose windows do not overlap (stride = window, no padding,
// no dilation: the pooling layers).  Every input pixel belongs to exactly one window, so a lane
// reads one vector of gradOut, scales it by the weight of its position in the window and writes
// one vector of gradIn: a plain stream.  The general gather would issue KH*KW masked loads per lane.
struct WindowArgs {
    const float *gradOut, *w;
    float *gradIn;
    int H, W, OH, OW, T, KW, P;  // P = H*W*T/VEC vectors per batch item
    int chunks;
    FastDiv byChunks, byTV, byW, bySH, bySW;
};

template <int VEC>
__global__ __launch_bounds__(256) void synapse_window_bwd_kernel(WindowArgs g)
{
    const uint32_t blk = xcd_contiguous(blockIdx.x, gridDim.x);
    const uint32_t n = fastdiv(blk, g.byChunks);
    const int p = static_cast<int>(blk - n * g.byChunks.d) * 256 + static_cast<int>(threadIdx.x);
    if (p >= g.P) return;
    const uint32_t pix = fastdiv(static_cast<uint32_t>(p), g.byTV);
    const int tv = p - static_cast<int>(pix * g.byTV.d);
    const int y = static_cast<int>(fastdiv(pix, g.byW)), x = static_cast<int>(pix) - y * g.W;
    const int a = static_cast<int>(fastdiv(static_cast<uint32_t>(y), g.bySH));
    const int b = static_cast<int>(fastdiv(static_cast<uint32_t>(x), g.bySW));
    const int i = y - a * static_cast<int>(g.bySH.d), j = x - b * static_cast<int>(g.bySW.d);
    const bool inside = a < g.OH && b < g.OW;  // rows and columns past the last whole window get no gradient
    const BufferRsrc src = make_buffer(g.gradOut + static_cast<int64_t>(n) * g.OH * g.OW * g.T);
    const BufferRsrc dst = make_buffer(g.gradIn + static_cast<int64_t>(n) * g.H * g.W * g.T);
    TimeVec<VEC> v, out;
    v.load(src, masked_offset(inside, ((a * g.OW + b) * g.T + tv * VEC) * 4));
    out.zero();
    out.fma(inside ? g.w[i * g.KW + j] : 0.f, v);
    out.store(dst, p * VEC * 4);
}

// ---- weight gradient -----------------------------------------------------------------------------
// gradW[o][c'][i][j] = sum_{n,a,b,t} gradOut[n][o][a][b][t] * in[n][c][a*sH-pH+i*dH][b*sW-pW+j*dW][t]
// A work-group owns OBW output channels x TAPS taps of one input channel for one slice of one batch
// item's (a, b, t) volume; a lane walks the slice's vectors with stride 256 keeping OBW x TAPS
// partial sums in registers.  The 256 lane sums are combined in a fixed tree (wavefront shuffles,
// then LDS) and written to a workspace row per slice; a second kernel adds the rows in order, so the
// result does not depend on scheduling.
struct WgradArgs {
    const float *gradOut, *in;
    float *partial;  // [slices][nW]
    SynGeom s;
    int Cg, Og, oBlocks, tapBlocks, slicesPerItem, P, perSlice;  // P = OH*OW*T/VEC vectors per plane
    FastDiv bySlices, byTapBlocks, byCg, byOBlocks, byGroups, byTV, byOW;
    int nW;
};

template <int OBW, int TAPS, int VEC>
__global__ __launch_bounds__(256) void synapse_wgrad_kernel(WgradArgs g)
{
    __shared__ float red[4][OBW * TAPS];
    const SynGeom &s = g.s;

    // all (channel block, channel, tap block) combinations of one slice are neighbours: they read
    // the same samples of gradOut and in
    uint32_t r = xcd_contiguous(blockIdx.x, gridDim.x);
    uint32_t q = fastdiv(r, g.byTapBlocks);
    const int tap0 = static_cast<int>(r - q * g.byTapBlocks.d) * TAPS;
    r = q; q = fastdiv(r, g.byCg);
    const int cl = static_cast<int>(r - q * g.byCg.d);
    r = q; q = fastdiv(r, g.byOBlocks);
    const int ol0 = static_cast<int>(r - q * g.byOBlocks.d) * OBW;
    r = q; q = fastdiv(r, g.byGroups);
    const int grp = static_cast<int>(r - q * g.byGroups.d);
    r = q; q = fastdiv(r, g.bySlices);
    const int slice = static_cast<int>(r - q * g.bySlices.d);
    const int n = static_cast<int>(q);

    const int KK = s.KH * s.KW;
    const int64_t goPlane = static_cast<int64_t>(s.OH) * s.OW * s.T, inPlane = static_cast<int64_t>(s.H) * s.W * s.T;
    const BufferRsrc goB = make_buffer(g.gradOut + (static_cast<int64_t>(n) * s.O + grp * g.Og + ol0) * goPlane);
    const BufferRsrc inB = make_buffer(g.in + (static_cast<int64_t>(n) * s.C + grp * g.Cg + cl) * inPlane);
    const int goPlaneBytes = static_cast<int>(goPlane) * 4;
    const int rowBytes = s.W * s.T * 4, pixBytes = s.T * 4;

    // tap offsets of this block (wave-uniform)
    int dy[TAPS], dx[TAPS];
#pragma unroll
    for (int k = 0; k < TAPS; ++k) {
        const int tap = tap0 + k;
        const int i = tap / s.KW, j = tap - i * s.KW;
        dy[k] = tap < KK ? i * s.dH - s.pH : -(1 << 28);  // a tap past the filter never lands inside
        dx[k] = j * s.dW - s.pW;
    }

    float acc[OBW][TAPS];
#pragma unroll
    for (int o = 0; o < OBW; ++o)
#pragma unroll
        for (int k = 0; k < TAPS; ++k) acc[o][k] = 0.f;

    const int pEnd = min(g.P, (slice + 1) * g.perSlice);
    for (int p = slice * g.perSlice + static_cast<int>(threadIdx.x); p < pEnd; p += 256) {
        const uint32_t pix = fastdiv(static_cast<uint32_t>(p), g.byTV);
        const int tv = p - static_cast<int>(pix * g.byTV.d);
        const int a = static_cast<int>(fastdiv(pix, g.byOW));
        const int b = static_cast<int>(pix) - a * s.OW;
        TimeVec<VEC> go[OBW];
#pragma unroll
        for (int o = 0; o < OBW; ++o) go[o].load(goB, masked_offset(ol0 + o < g.Og, o * goPlaneBytes + p * VEC * 4));
        const int y0 = a * s.sH, x0 = b * s.sW, laneBytes = tv * VEC * 4;
#pragma unroll
        for (int k = 0; k < TAPS; ++k) {
            const int y = y0 + dy[k], x = x0 + dx[k];
            const bool ok = static_cast<unsigned>(y) < static_cast<unsigned>(s.H) &&
                            static_cast<unsigned>(x) < static_cast<unsigned>(s.W);
            TimeVec<VEC> xv;
            xv.load(inB, masked_offset(ok, y * rowBytes + x * pixBytes + laneBytes));
#pragma unroll
            for (int o = 0; o < OBW; ++o) acc[o][k] = go[o].dot(xv, acc[o][k]);
        }
    }

    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
    for (int o = 0; o < OBW; ++o)
#pragma unroll
        for (int k = 0; k < TAPS; ++k) {
            float v = acc[o][k];
#pragma unroll
            for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_down(v, off, kWave);
            if (lane == 0) red[wave][o * TAPS + k] = v;
        }
    __syncthreads();
    if (threadIdx.x < OBW * TAPS) {
        const int o = threadIdx.x / TAPS, k = threadIdx.x - o * TAPS;
        if (ol0 + o < g.Og && tap0 + k < KK) {
            const float v = ((red[0][threadIdx.x] + red[1][threadIdx.x]) + red[2][threadIdx.x]) + red[3][threadIdx.x];
            const int64_t widx = (static_cast<int64_t>(grp * g.Og + ol0 + o) * g.Cg + cl) * KK + tap0 + k;
            g.partial[(static_cast<int64_t>(n) * g.slicesPerItem + slice) * g.nW + widx] = v;
        }
    }
}


// ---- weight gradient on the matrix cores ------------------------------------------------------
// For one output pixel (n, a, b) the weight gradient is a matrix product with time as the
// reduction axis:  gradW[o][col] += sum_t G[o][t] * X[col][t],  G[o][t] = gradOut[n][o][a][b][t],
// X[col][t] = in[n][c][a*sH-pH+i*dH][b*sW-pW+j*dW][t] for col = (c, i, j).  Both operands are rows
// that are contiguous in t, which is exactly the register layout of v_mfma_f32_16x16x4_f32: lane
// (r, h) = (lane % 16, lane / 16) supplies row r at reduction index h of both operands.  A lane
// loads 16 bytes - four time samples t = 16*step + 4*h + e - and feeds them to four matrix
// instructions (e = 0..3); the order in which time samples enter the sum does not matter as long
// as both operands use the same one.  A 16-lane group reads 64 contiguous bytes of each of 16 rows,
// so every byte a load instruction fetches is used and the operands need no staging in LDS.
// A wavefront owns MT x NT tiles of 16 output channels x 16 columns; the four wavefronts of a
// work-group take neighbouring pixels of a slice of one batch item at the same time (their input
// rows overlap, so they share them through the L1 cache), add their tiles up in LDS in wavefront
// order and write one workspace row per slice.
typedef float floatx4 __attribute__((ext_vector_type(4)));

struct WgradMfmaArgs {
    const float *gradOut, *in;
    float *partial;
    SynGeom s;
    int Cg, Og, CK;          // input channels, output channels and columns (Cg * KH * KW) per group
    int oGroups, colGroups;  // blocks of 16*MT output channels / 16*NT columns per group
    int slices, pixPerSlice, nW;
    FastDiv bySlices, byColGroups, byOGroups, byGroups, byKK, byKW, byOW;
};

template <int MT, int NT>
__global__ __launch_bounds__(256) void synapse_wgrad_mfma_kernel(WgradMfmaArgs g)
{
    __shared__ float red[MT * NT * 256];
    const SynGeom &s = g.s;
    // the tile groups of one slice of pixels are neighbours: they read the same operand rows
    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    uint32_t q = fastdiv(rest, g.byColGroups);
    const int cg = static_cast<int>(rest - q * g.byColGroups.d);
    rest = q; q = fastdiv(rest, g.byOGroups);
    const int og = static_cast<int>(rest - q * g.byOGroups.d);
    rest = q; q = fastdiv(rest, g.byGroups);
    const int grp = static_cast<int>(rest - q * g.byGroups.d);
    rest = q; q = fastdiv(rest, g.bySlices);
    const int slice = static_cast<int>(rest - q * g.bySlices.d);
    const int n = static_cast<int>(q);

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, r = lane & 15, h = lane >> 4;
    const int64_t goPlane = static_cast<int64_t>(s.OH) * s.OW * s.T, inPlane = static_cast<int64_t>(s.H) * s.W * s.T;
    const BufferRsrc goB = make_buffer(g.gradOut + (static_cast<int64_t>(n) * s.O + grp * g.Og) * goPlane);
    const BufferRsrc inB = make_buffer(g.in + (static_cast<int64_t>(n) * s.C + grp * g.Cg) * inPlane);
    const int rowBytes = s.W * s.T * 4, pixBytes = s.T * 4;

    // rows of this lane: output channel of every A tile, (channel, tap) of every B tile
    int offA[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int o = ((og * MT + mt) << 4) + r;
        offA[mt] = masked_offset(o < g.Og, o * static_cast<int>(goPlane) * 4);
    }
    int baseB[NT], dyB[NT], dxB[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int col = ((cg * NT + nt) << 4) + r;
        const uint32_t cl = fastdiv(static_cast<uint32_t>(col), g.byKK);
        const int ij = col - static_cast<int>(cl * g.byKK.d);
        const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(ij), g.byKW));
        const int j = ij - i * s.KW;
        baseB[nt] = col < g.CK ? static_cast<int>(cl) * static_cast<int>(inPlane) * 4 : 0;
        dyB[nt] = col < g.CK ? i * s.dH - s.pH : -(1 << 28);  // a column past the filter never lands inside
        dxB[nt] = j * s.dW - s.pW;
    }

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};

    const int steps = (s.T + 15) >> 4;
    const int pixEnd = min(s.OH * s.OW, (slice + 1) * g.pixPerSlice);
    int offB[NT];
    auto place = [&](int pixel) {  // byte offsets of this lane's B rows for an output pixel
        const int a = static_cast<int>(fastdiv(static_cast<uint32_t>(pixel), g.byOW));
        const int b = pixel - a * s.OW;
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const int y = a * s.sH + dyB[nt], x = b * s.sW + dxB[nt];
            const bool ok = static_cast<unsigned>(y) < static_cast<unsigned>(s.H) &&
                            static_cast<unsigned>(x) < static_cast<unsigned>(s.W);
            offB[nt] = masked_offset(ok, baseB[nt] + y * rowBytes + x * pixBytes);
        }
    };
    // an offset that is already out of range stays out of range when a small number is added
    auto issue = [&](float4 (&A)[MT], float4 (&B)[NT], int pixel, int st, bool more) {
        const int t = (st << 4) + (h << 2);
        const bool live = more && t < s.T;
        const int pixA = pixel * pixBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
            A[mt] = buffer_load4<0>(goB, live && offA[mt] != kOutOfRange ? offA[mt] + pixA + t * 4 : kOutOfRange, 0);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            B[nt] = buffer_load4<0>(inB, live && offB[nt] != kOutOfRange ? offB[nt] + t * 4 : kOutOfRange, 0);
    };

    // (pixel, step) pairs in order; the operands of the next pair are loaded while the matrix
    // instructions of the current one run
    int pixel = slice * g.pixPerSlice + wave, st = 0;
    if (pixel < pixEnd) {
        float4 A[MT], B[NT];
        place(pixel);
        issue(A, B, pixel, st, true);
        for (;;) {
            int nst = st + 1, npix = pixel;
            if (nst == steps) {
                nst = 0;
                npix += 4;
                if (npix < pixEnd) place(npix);
            }
            const bool more = npix < pixEnd;
            float4 An[MT], Bn[NT];
            issue(An, Bn, npix, nst, more);
            // consecutive matrix instructions go to different accumulators
#define SLAYER_WGRAD_MFMA(E)                                                                              \
    _Pragma("unroll") for (int mt = 0; mt < MT; ++mt) _Pragma("unroll") for (int nt = 0; nt < NT; ++nt)     \
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(A[mt].E, B[nt].E, acc[mt][nt], 0, 0, 0);
            SLAYER_WGRAD_MFMA(x)
            SLAYER_WGRAD_MFMA(y)
            SLAYER_WGRAD_MFMA(z)
            SLAYER_WGRAD_MFMA(w)
#undef SLAYER_WGRAD_MFMA
            if (!more) break;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) A[mt] = An[mt];
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) B[nt] = Bn[nt];
            pixel = npix;
            st = nst;
        }
    }

    // the four wavefronts add their tiles in LDS, in wavefront order
    for (int w = 0; w < 4; ++w) {
        if (wave == w) {
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                    for (int v = 0; v < 4; ++v) {
                        float *cell = red + ((mt * NT + nt) * 4 + v) * 64 + lane;
                        *cell = w == 0 ? acc[mt][nt][v] : *cell + acc[mt][nt][v];
                    }
        }
        __syncthreads();
    }
    // element v of a tile's accumulator is row 4*h + v, column r of the tile
    float *row = g.partial + (static_cast<int64_t>(n) * g.slices + slice) * g.nW;
    for (int e = threadIdx.x; e < MT * NT * 256; e += 256) {
        const int tile = e >> 8, v = (e >> 6) & 3, l = e & 63;
        const int mt = tile / NT, nt = tile - mt * NT;
        const int o = ((og * MT + mt) << 4) + ((l >> 4) << 2) + v;
        const int col = ((cg * NT + nt) << 4) + (l & 15);
        if (o < g.Og && col < g.CK) row[static_cast<int64_t>(grp * g.Og + o) * g.CK + col] = red[e];
    }
}

// ---- gather on the matrix cores --------------------------------------------------------------------------
// For 16 output channels and 16 time samples of one pixel, dst[t][o] = sum_k X[k][t] * W[k][o] over the taps
// k = (source channel, filter row, filter column) is a matrix product with the taps as the reduction axis:
// v_mfma_f32_16x16x4_f32 takes four taps at a time, lane (r, h) supplying X[k0 + h][t0 + r] and W[k0 + h][o0 + r],
// and leaves four consecutive time samples of channel o0 + r in its accumulator - one 16-byte store.  A
// work-group of eight wavefronts takes kGmPix = 8 consecutive destination pixels of one row (one per wavefront)
// and a step of 32 time samples at a time and copies the source patch under those pixels into LDS once - up to
// 16 source channels ("a pass") x KH filter rows x WX columns, one whole 128-byte line each, out-of-image
// positions as zeros - so the X operands are one LDS dword per matrix instruction at an address that is the
// same in every step (a table of 36 registers per lane; the half of the step and the buffer are immediates).  The weights of all passes sit in LDS as
// [pass][channel tile][lane][tap step], a lane's steps contiguous: one 16-byte read per four steps.  Two
// patches are resident; the loads of the next (pixel block, step, pass) are in flight in registers while the
// matrix instructions work, and are written to the other patch before the single barrier.  Source channels
// beyond a pass are accumulated by running the passes of a (block, step) one after the other; the accumulators
// leave after the last.  Work is cut into equal ranges of (block, step) pairs of the whole batch, one
// work-group per compute unit (its LDS).
constexpr int kGmPix = 8;
constexpr int kGmRow = 128;                    // bytes per patch row: 32 samples
constexpr int kGmMaxRows = 480;                // patch rows; row kGmMaxRows of a buffer holds zeros
constexpr int kGmBuf = (kGmMaxRows + 1) * kGmRow;
constexpr int kGmSteps = 36;                   // tap steps per pass: 144 taps (16 channels x 3 x 3)
constexpr int kGmMaxWeightBytes = 4 * 64 * kGmSteps * 4;   // passes x channel tiles <= 4

struct GatherMfmaArgs {
    const float *src;
    float *dst;
    const float *w;
    int SC, SH, SW, DC, DH, DW, T;
    int Qg, Mg, groups, KH, KW, Cg, Og;
    int mulH, mulW, offH, offW, stepH, stepW;
    int chansPerPass, passes, WX, xBias, rows;   // patch: chansPerPass x KH x WX rows; xBias: patch column of tap 0 of pixel 0
    int oGroups;                                 // blocks of 16 * OT destination channels per group
    int blocksPerRow, steps, pairs, slices, pairsPerSlice;
    FastDiv byOGroups, byGroups, byKK, byKW, bySteps, byBlocks, byBlocksPerRow, byPatch, byWX;
};

template <int OT, bool BACKWARD>
__global__ __launch_bounds__(512) void synapse_gather_mfma_kernel(GatherMfmaArgs g)
{
    extern __shared__ __align__(16) float lds[];
    char *const ldsBytes = reinterpret_cast<char *>(lds);
    constexpr int KS = kGmSteps;
    // (LDS addresses as plain 32-bit numbers: the tables below then hold final addresses, nothing is added per read)
    typedef const float __attribute__((address_space(3))) *LdsFloat;
    typedef const floatx4 __attribute__((address_space(3))) *LdsFloat4;
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char *)ldsBytes));
    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    uint32_t qq = fastdiv(rest, g.byOGroups);
    const int og = static_cast<int>(rest - qq * g.byOGroups.d);
    rest = qq; qq = fastdiv(rest, g.byGroups);
    const int grp = static_cast<int>(rest - qq * g.byGroups.d);
    const int slice = static_cast<int>(qq);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, h = lane >> 4;
    const int KK = g.KH * g.KW;
    const int64_t srcPlane = static_cast<int64_t>(g.SH) * g.SW * g.T, dstPlane = static_cast<int64_t>(g.DH) * g.DW * g.T;
    const int rowBytes = g.SW * g.T * 4, pixBytes = g.T * 4, planeBytes = static_cast<int>(srcPlane) * 4;
    BufferRsrc srcB = make_buffer(g.src), dstB = make_buffer(g.dst);   // (of the batch item at hand: set by place())

    // weights: wl[((pass * OT + ot) * 64 + lane) * KS + s] = W[tap 4 s + h of the pass][channel 16 (og OT + ot) + r]
    float *const wl = lds + 2 * kGmBuf / 4;   // (behind the two patches and their zero rows)
    for (int e = tid; e < g.passes * OT * 64 * KS; e += 512) {
        const int s = e % KS, l = (e / KS) & 63, po = e / (KS * 64);
        const int ot = po % OT, pass = po / OT;
        const int k = 4 * s + (l >> 4), m = (og * OT + ot) * 16 + (l & 15);
        const int cl = static_cast<int>(fastdiv(static_cast<uint32_t>(k), g.byKK)), ij = k - cl * KK, q = pass * g.chansPerPass + cl;
        float v = 0.f;
        if (cl < g.chansPerPass && q < g.Qg && m < g.Mg) {
            const int64_t idx = BACKWARD ? (static_cast<int64_t>(grp * g.Og + q) * g.Cg + m) * KK + ij
                                         : (static_cast<int64_t>(grp * g.Og + m) * g.Cg + q) * KK + ij;
            v = g.w[idx];
        }
        wl[e] = v;
    }
    if (tid < 2 * (kGmRow / 4)) lds[kGmMaxRows * 2 * kGmRow / 4 + tid] = 0.f;   // the zero rows of both patches

    // X operand of tap step s: LDS address of this lane's sample in the first half of the step's 32 samples (the
    // second half lies 64 bytes on, the other patch kGmBuf bytes on: immediates).  Patch rows are not swizzled
    // here: a read takes 64 contiguous bytes of each of 4 rows, at worst two of them in the same banks.  The rows
    // of the two patches alternate (row r of patch b at (2 r + b) * 128 bytes), so that the patch, too, is an
    // immediate within reach of a two-address LDS read.
    int aTab[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int k = 4 * s + h;
        const uint32_t cl = fastdiv(static_cast<uint32_t>(k), g.byKK);
        const int ij = k - static_cast<int>(cl * g.byKK.d);
        const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(ij), g.byKW));
        const int j = ij - i * g.KW;
        const int row = static_cast<int>(cl) < g.chansPerPass
            ? (static_cast<int>(cl) * g.KH + i) * g.WX + wave * g.mulW + j * g.stepW + g.xBias : kGmMaxRows;
        aTab[s] = static_cast<int>(ldsBase) + row * 2 * kGmRow + (r << 2);
    }
    const uint32_t wAddr = ldsBase + 2 * kGmBuf + lane * KS * 4;

    // destination rows of this lane: channel 16 (og OT + ot) + r, samples 4 h .. 4 h + 3 of a half step
    int oOff[OT];
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
        const int m = (og * OT + ot) * 16 + r;
        oOff[ot] = masked_offset(m < g.Mg, m * static_cast<int>(dstPlane) * 4 + h * 16);
    }

    // This lane copies unit u (samples 4u..4u+3 of the step) of patch rows tid / 8 + 64 m
    constexpr int NS = 8;
    const int u = tid & 7;
    const int stageAddr = (tid >> 3) * 2 * kGmRow + (u << 4);

    const int p0 = slice * g.pairsPerSlice, p1 = min(g.pairs, p0 + g.pairsPerSlice);
    int sOff[NS];
    int pixNext = 0;          // byte offset of this wavefront's destination pixel in a channel plane, or -1
    auto place = [&](int blockOfAll) {
        const int n = static_cast<int>(fastdiv(static_cast<uint32_t>(blockOfAll), g.byBlocks));
        const int block = blockOfAll - n * static_cast<int>(g.byBlocks.d);
        srcB = make_buffer(g.src + (static_cast<int64_t>(n) * g.SC + static_cast<int64_t>(grp) * g.Qg) * srcPlane);
        const int a = static_cast<int>(fastdiv(static_cast<uint32_t>(block), g.byBlocksPerRow));
        const int b0 = (block - a * g.blocksPerRow) * kGmPix;
        const int nv = min(kGmPix, g.DW - b0);
        const int xLimit = (nv - 1) * g.mulW + (g.KW - 1) * (g.stepW < 0 ? -g.stepW : g.stepW) + 1;
        const int y0 = a * g.mulH + g.offH, x0 = b0 * g.mulW + g.offW - g.xBias;
#pragma unroll
        for (int m = 0; m < NS; ++m) {
            const int row = (tid >> 3) + 64 * m;
            const uint32_t cl = fastdiv(static_cast<uint32_t>(row), g.byPatch);
            const int rem = row - static_cast<int>(cl * g.byPatch.d);
            const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(rem), g.byWX));
            const int x = rem - i * g.WX;
            const int y = y0 + i * g.stepH, xx = x0 + x;
            const bool ok = row < g.rows && x < xLimit && static_cast<unsigned>(y) < static_cast<unsigned>(g.SH) &&
                            static_cast<unsigned>(xx) < static_cast<unsigned>(g.SW);
            sOff[m] = masked_offset(ok, static_cast<int>(cl) * planeBytes + y * rowBytes + xx * pixBytes + u * 16);
        }
        const int b = b0 + wave;
        pixNext = b < g.DW ? (a * g.DW + b) * pixBytes : -1;
        return n;
    };
    auto issue = [&](float4 (&R)[NS], int st, int pass, bool more) {
        const int uniform = (st << 7) + pass * g.chansPerPass * planeBytes;
        const bool live = more && (st << 5) + (u << 2) < g.T;
#pragma unroll
        for (int m = 0; m < NS; ++m) R[m] = buffer_load4<0>(srcB, live ? sOff[m] : kOutOfRange, uniform);
    };
    auto stage = [&](const float4 (&R)[NS], int buf) {
#pragma unroll
        for (int m = 0; m < NS; ++m)
            if ((tid >> 3) + 64 * m < kGmMaxRows) *reinterpret_cast<float4 *>(ldsBytes + buf + stageAddr + m * 64 * 2 * kGmRow) = R[m];
    };

    floatx4 acc[2][OT];
    auto clear = [&]() {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int ot = 0; ot < OT; ++ot) acc[hf][ot] = floatx4{0.f, 0.f, 0.f, 0.f};
    };
    // the matrix work of one pass on the patch in buffer BUF (an immediate in every LDS read); HALVES = 1 when the
    // second half of the step lies past the end of the row.  Straight-line code: the LDS reads run ahead of the
    // matrix instructions that use them.
    auto multiply = [&](auto bufTag, auto halvesTag, int pass) {
        constexpr int BUF = decltype(bufTag)::value, HALVES = decltype(halvesTag)::value;
        const uint32_t wp = wAddr + pass * OT * 64 * KS * 4;
        // operands of four tap steps at a time, fetched one group ahead of the matrix instructions that use them
        floatx4 bq[2][OT];
        float av[2][HALVES][4];
        auto fetch = [&](int set, int s4) {
#pragma unroll
            for (int ot = 0; ot < OT; ++ot)
                bq[set][ot] = *reinterpret_cast<LdsFloat4>(static_cast<size_t>(wp + (ot * 64 * KS + s4) * 4));
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int hf = 0; hf < HALVES; ++hf)
                    av[set][hf][e] = *reinterpret_cast<LdsFloat>(static_cast<size_t>(static_cast<uint32_t>(aTab[s4 + e]) + BUF * kGmRow + hf * 64));
        };
        fetch(0, 0);
#pragma unroll
        for (int s4 = 0; s4 < KS; s4 += 4) {
            const int set = (s4 >> 2) & 1;
            if (s4 + 4 < KS) fetch(set ^ 1, s4 + 4);
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int hf = 0; hf < HALVES; ++hf)
#pragma unroll
                    for (int ot = 0; ot < OT; ++ot)
                        acc[hf][ot] = __builtin_amdgcn_mfma_f32_16x16x4f32(av[set][hf][e], bq[set][ot][e], acc[hf][ot], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // the accumulators of a (block, step) leave: four consecutive samples of one channel per lane and tile.  A store
    // instruction writes 64 bytes of each of 16 channel rows, and a pixel's row is 4 T bytes long: cached stores, so
    // that L2 puts the pieces of a line together (streaming stores of these pieces: 137 us instead of 114 us on
    // the 16 -> 32 channel layer)
    auto store = [&](int pix, int st) {
        if (pix < 0) return;
        const int uniform = pix + (st << 7);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const bool live = (st << 5) + hf * 16 + (h << 2) < g.T;
#pragma unroll
            for (int ot = 0; ot < OT; ++ot)
                buffer_store4<0>(dstB, live ? oOff[ot] : kOutOfRange, uniform + hf * 64,
                                       make_float4(acc[hf][ot][0], acc[hf][ot][1], acc[hf][ot][2], acc[hf][ot][3]));
        }
    };

    {
        // Trip k of the loop loads (pair, pass) number k of the range into registers, multiplies number k - 1 from
        // its LDS buffer ((k - 1) % 2) and then writes the registers to the other buffer: the loop's code exists
        // once, its first trip only loads.
        // Pairs are numbered with the pixel block fastest, then the step, then the batch item: consecutive pairs of
        // a range are neighbouring patches of the same 32 samples, whose shared rows and columns come from L2
        // instead of from memory (with the step fastest every pair fetched all of its patch from beyond L2: 4.7 x
        // the source tensor on the 16 -> 32 channel layer, 6 x in its input gradient).
        const int perItem = static_cast<int>(g.byBlocks.d);   // pixel blocks of a batch item
        int image = static_cast<int>(fastdiv(static_cast<uint32_t>(p0), g.byBlocks));
        int inItem = p0 - image * perItem;                // pixel block within the batch item ..
        int item = static_cast<int>(fastdiv(static_cast<uint32_t>(image), g.bySteps));
        int st = image - item * g.steps, pass = 0;        // .. step and pass that are loaded next
        int stCur = 0, passCur = 0, pixCur = -1, nCur = -1, nNext = -1;   // what is multiplied next
        float4 R[NS];
        int buf = 1;
        bool first = true;
        const int trips = (p1 - p0) * g.passes;
        clear();
#pragma nounroll
        for (int k = 0;; ++k) {
            const bool more = k < trips;
            bool moved = first;
            if (more && !first) {
                if (++pass == g.passes) {
                    pass = 0;
                    moved = true;
                    if (++inItem == perItem) {
                        inItem = 0;
                        if (++st == g.steps) {
                            st = 0;
                            ++item;
                        }
                    }
                }
            }
            if (more && moved) nNext = place(item * perItem + inItem);
            issue(R, st, pass, more);
            __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the matrix work
            if (!first) {
                using I0 = std::integral_constant<int, 0>;
                using I1 = std::integral_constant<int, 1>;
                using I2 = std::integral_constant<int, 2>;
                if ((stCur << 5) + 16 < g.T) {
                    if (buf == 0) multiply(I0{}, I2{}, passCur);
                    else multiply(I1{}, I2{}, passCur);
                } else {
                    if (buf == 0) multiply(I0{}, I1{}, passCur);
                    else multiply(I1{}, I1{}, passCur);
                }
                if (passCur == g.passes - 1) {
                    if (nCur >= 0) {
                        dstB = make_buffer(g.dst + (static_cast<int64_t>(nCur) * g.DC + static_cast<int64_t>(grp) * g.Mg) * dstPlane);
                        store(pixCur, stCur);
                    }
                    clear();
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!more) break;
            buf ^= 1;
            stage(R, buf * kGmRow);
            stCur = st; passCur = pass; pixCur = pixNext; nCur = nNext;
            __syncthreads();
            first = false;
        }
    }
}

// ---- gather on the matrix cores, bf16 instructions over split operands ---------------------------------------
// The same work-group, patch and loop as above, with v_mfma_f32_16x16x32_bf16 in place of the fp32 instruction: 32
// taps per instruction in half the time of the fp32 instruction's four.  Every fp32 number is the sum of three bf16
// numbers (its upper 16 bits, those of the remainder, and those of what is left), so a product of two is the sum
// of nine partial products, of which the six largest are kept (the error, below 2^-22 of |x| |w| per term, is that
// of the fp32 sum itself).  The weights are split once per work-group, in LDS in the register layout of the
// instruction's second operand ([pass][channel tile][group of 32 taps][part][lane], 16 bytes each).  The patch
// stays fp32: lane (r, h) reads its sample r of the 8 taps 32 G + 8 h .. + 7 as eight dwords and splits them in
// registers - or only packs their upper halves when the patch holds nothing else, which the staging wavefronts
// note per patch (spike tensors: 0 and 1 / Ts with few significant bits): three products instead of six.
// A pass has room for 5 groups (160 taps >= the 144 of a pass; taps beyond the pass read the zero row and carry zero
// weights).  With at most two (pass, channel tile) sets of weights the two patches of the kernel above fit beside
// them; with up to four there is one patch, written between two barriers after the matrix work.  Numbers below
// 2^-126 in a part are flushed by the instruction; a non-finite input sample gives NaN where the fp32 sum may
// give an infinity.
constexpr int kGsGroups = 5;
constexpr int kGsUnitBytes = kGsGroups * 3 * 1024;      // weights of one (pass, channel tile)

template <int OT, bool BACKWARD, bool DOUBLE>
__global__ __launch_bounds__(512) void synapse_gather_split_kernel(GatherMfmaArgs g)
{
    extern __shared__ __align__(16) float lds[];
    char *const ldsBytes = reinterpret_cast<char *>(lds);
    constexpr int NG = kGsGroups;
    constexpr int STRIDE = DOUBLE ? 2 * kGmRow : kGmRow;     // between patch rows (the rows of two patches alternate)
    constexpr int PATCH = DOUBLE ? 2 * kGmBuf : kGmBuf;
    typedef const float __attribute__((address_space(3))) *LdsFloat;
    typedef const uint4_ext __attribute__((address_space(3))) *LdsUint4;
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char *)ldsBytes));
    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    uint32_t qq = fastdiv(rest, g.byOGroups);
    const int og = static_cast<int>(rest - qq * g.byOGroups.d);
    rest = qq; qq = fastdiv(rest, g.byGroups);
    const int grp = static_cast<int>(rest - qq * g.byGroups.d);
    const int slice = static_cast<int>(qq);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, h = lane >> 4;
    const int KK = g.KH * g.KW;
    const int64_t srcPlane = static_cast<int64_t>(g.SH) * g.SW * g.T, dstPlane = static_cast<int64_t>(g.DH) * g.DW * g.T;
    const int rowBytes = g.SW * g.T * 4, pixBytes = g.T * 4, planeBytes = static_cast<int>(srcPlane) * 4;
    BufferRsrc srcB = make_buffer(g.src), dstB = make_buffer(g.dst);   // (of the batch item at hand: set by place())

    // weights: unit (pass, ot), group G, part, lane (r, h): taps 32 G + 8 h .. + 7 of the pass for channel
    // 16 (og OT + ot) + r
    uint4_ext *const wl = reinterpret_cast<uint4_ext *>(ldsBytes + PATCH);
    uint32_t *const flags = reinterpret_cast<uint32_t *>(ldsBytes + PATCH + g.passes * OT * kGsUnitBytes);   // [2][8]
    for (int e = tid; e < g.passes * OT * NG * 64; e += 512) {
        const int l = e & 63, G = (e >> 6) % NG, po = (e >> 6) / NG;
        const int ot = po % OT, pass = po / OT;
        const int m = (og * OT + ot) * 16 + (l & 15);
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int k = 32 * G + 8 * (l >> 4) + j;
            const int cl = static_cast<int>(fastdiv(static_cast<uint32_t>(k), g.byKK)), ij = k - cl * KK, q = pass * g.chansPerPass + cl;
            v[j] = 0.f;
            if (cl < g.chansPerPass && q < g.Qg && m < g.Mg) {
                const int64_t idx = BACKWARD ? (static_cast<int64_t>(grp * g.Og + q) * g.Cg + m) * KK + ij
                                             : (static_cast<int64_t>(grp * g.Og + m) * g.Cg + q) * KK + ij;
                v[j] = g.w[idx];
            }
        }
        const SplitPlanes sp = split_bf16(v);
        uint4_ext *unit = wl + (po * NG + G) * 3 * 64 + l;
        unit[0] = sp.hi;
        unit[64] = sp.mid;
        unit[128] = sp.lo;
    }
    if (tid < (DOUBLE ? 2 : 1) * (kGmRow / 4)) lds[kGmMaxRows * STRIDE / 4 + tid] = 0.f;   // the zero row of every patch

    // this lane's sample r (of the first half of a step; the second lies 64 bytes on) of tap 32 G + 8 h + e
    int aTab[NG][8];
#pragma unroll
    for (int G = 0; G < NG; ++G)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int k = 32 * G + 8 * h + e;
            const uint32_t cl = fastdiv(static_cast<uint32_t>(k), g.byKK);
            const int ij = k - static_cast<int>(cl * g.byKK.d);
            const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(ij), g.byKW));
            const int j = ij - i * g.KW;
            const int row = static_cast<int>(cl) < g.chansPerPass
                ? (static_cast<int>(cl) * g.KH + i) * g.WX + wave * g.mulW + j * g.stepW + g.xBias : kGmMaxRows;
            aTab[G][e] = static_cast<int>(ldsBase) + row * STRIDE + (r << 2);
        }
    const uint32_t wAddr = ldsBase + PATCH + lane * 16;

    int oOff[OT];
#pragma unroll
    for (int ot = 0; ot < OT; ++ot) {
        const int m = (og * OT + ot) * 16 + r;
        oOff[ot] = masked_offset(m < g.Mg, m * static_cast<int>(dstPlane) * 4 + h * 16);
    }

    // This lane copies unit u (samples 4u..4u+3 of the step) of patch rows tid / 8 + 64 m
    constexpr int NS = 8;
    const int u = tid & 7;
    const int stageAddr = (tid >> 3) * STRIDE + (u << 4);

    const int p0 = slice * g.pairsPerSlice, p1 = min(g.pairs, p0 + g.pairsPerSlice);
    int sOff[NS];
    int pixNext = 0;          // byte offset of this wavefront's destination pixel in a channel plane, or -1
    auto place = [&](int blockOfAll) {
        const int n = static_cast<int>(fastdiv(static_cast<uint32_t>(blockOfAll), g.byBlocks));
        const int block = blockOfAll - n * static_cast<int>(g.byBlocks.d);
        srcB = make_buffer(g.src + (static_cast<int64_t>(n) * g.SC + static_cast<int64_t>(grp) * g.Qg) * srcPlane);
        const int a = static_cast<int>(fastdiv(static_cast<uint32_t>(block), g.byBlocksPerRow));
        const int b0 = (block - a * g.blocksPerRow) * kGmPix;
        const int nv = min(kGmPix, g.DW - b0);
        const int xLimit = (nv - 1) * g.mulW + (g.KW - 1) * (g.stepW < 0 ? -g.stepW : g.stepW) + 1;
        const int y0 = a * g.mulH + g.offH, x0 = b0 * g.mulW + g.offW - g.xBias;
#pragma unroll
        for (int m = 0; m < NS; ++m) {
            const int row = (tid >> 3) + 64 * m;
            const uint32_t cl = fastdiv(static_cast<uint32_t>(row), g.byPatch);
            const int rem = row - static_cast<int>(cl * g.byPatch.d);
            const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(rem), g.byWX));
            const int x = rem - i * g.WX;
            const int y = y0 + i * g.stepH, xx = x0 + x;
            const bool ok = row < g.rows && x < xLimit && static_cast<unsigned>(y) < static_cast<unsigned>(g.SH) &&
                            static_cast<unsigned>(xx) < static_cast<unsigned>(g.SW);
            sOff[m] = masked_offset(ok, static_cast<int>(cl) * planeBytes + y * rowBytes + xx * pixBytes + u * 16);
        }
        const int b = b0 + wave;
        pixNext = b < g.DW ? (a * g.DW + b) * pixBytes : -1;
        return n;
    };
    auto issue = [&](float4 (&R)[NS], int st, int pass, bool more) {
        const int uniform = (st << 7) + pass * g.chansPerPass * planeBytes;
        const bool live = more && (st << 5) + (u << 2) < g.T;
#pragma unroll
        for (int m = 0; m < NS; ++m) R[m] = buffer_load4<0>(srcB, live ? sOff[m] : kOutOfRange, uniform);
    };
    // registers -> patch; a wavefront notes whether any of its samples has more than the upper 16 bits
    auto stage = [&](const float4 (&R)[NS], int buf) {
        uint32_t low = 0;
#pragma unroll
        for (int m = 0; m < NS; ++m) {
            if ((tid >> 3) + 64 * m < kGmMaxRows) *reinterpret_cast<float4 *>(ldsBytes + buf * kGmRow + stageAddr + m * 64 * STRIDE) = R[m];
            low |= (__builtin_bit_cast(uint32_t, R[m].x) | __builtin_bit_cast(uint32_t, R[m].y)) |
                   (__builtin_bit_cast(uint32_t, R[m].z) | __builtin_bit_cast(uint32_t, R[m].w));
        }
        const bool any = __builtin_amdgcn_ballot_w64((low & 0xffffu) != 0u) != 0;
        if (lane == 0) flags[buf * 8 + wave] = any ? 1u : 0u;
    };

    f32x4 acc[2][OT];
    auto clear = [&]() {
#pragma unroll
        for (int hf = 0; hf < 2; ++hf)
#pragma unroll
            for (int ot = 0; ot < OT; ++ot) acc[hf][ot] = f32x4{0.f, 0.f, 0.f, 0.f};
    };
    // the matrix work of one pass on the patch in buffer BUF; HALVES = 1 when the second half of the step lies past
    // the end of the row.  The samples of a group of taps are read while the group before is multiplied.
    auto multiply = [&](auto bufTag, auto halvesTag, int pass, int buf) {
        constexpr int BUF = decltype(bufTag)::value, HALVES = decltype(halvesTag)::value;
        const bool allParts = __builtin_amdgcn_ballot_w64(lane < 8 && flags[buf * 8 + (lane & 7)] != 0u) != 0;
        const uint32_t wp = wAddr + pass * OT * kGsUnitBytes;
        uint4_ext wq[OT][3];
        float av[2][HALVES][8];
        auto fetch = [&](int set, int G) {
#pragma unroll
            for (int hf = 0; hf < HALVES; ++hf)
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    av[set][hf][e] = *reinterpret_cast<LdsFloat>(static_cast<size_t>(static_cast<uint32_t>(aTab[G][e]) + BUF * kGmRow + hf * 64));
        };
        fetch(0, 0);
#pragma unroll
        for (int G = 0; G < NG; ++G) {
            const int set = G & 1;
            // (the weights of this group, then the samples of the next: a second set of weights a group ahead does
            // not fit the registers)
#pragma unroll
            for (int ot = 0; ot < OT; ++ot)
#pragma unroll
                for (int part = 0; part < 3; ++part)
                    wq[ot][part] = *reinterpret_cast<LdsUint4>(static_cast<size_t>(wp + ((ot * NG + G) * 3 + part) * 1024));
            if (G + 1 < NG) fetch(set ^ 1, G + 1);
            __builtin_amdgcn_sched_barrier(0);   // (issued here, ahead of the matrix instructions of this group)
            if (allParts) {
#pragma unroll
                for (int hf = 0; hf < HALVES; ++hf) {
                    const SplitPlanes a = split_bf16(av[set][hf]);
#pragma unroll
                    for (int ot = 0; ot < OT; ++ot) {
                        acc[hf][ot] = mfma_bf16(a.hi, wq[ot][2], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a.lo, wq[ot][0], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a.mid, wq[ot][1], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a.hi, wq[ot][1], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a.mid, wq[ot][0], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a.hi, wq[ot][0], acc[hf][ot]);
                    }
                }
            } else {
#pragma unroll
                for (int hf = 0; hf < HALVES; ++hf) {
                    uint4_ext a;
#pragma unroll
                    for (int w2 = 0; w2 < 4; ++w2)
                        a[w2] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, av[set][hf][2 * w2 + 1]),
                                                      __builtin_bit_cast(uint32_t, av[set][hf][2 * w2]), 0x07060302u);
#pragma unroll
                    for (int ot = 0; ot < OT; ++ot) {
                        acc[hf][ot] = mfma_bf16(a, wq[ot][2], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a, wq[ot][1], acc[hf][ot]);
                        acc[hf][ot] = mfma_bf16(a, wq[ot][0], acc[hf][ot]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto store = [&](int pix, int st) {
        if (pix < 0) return;
        const int uniform = pix + (st << 7);
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const bool live = (st << 5) + hf * 16 + (h << 2) < g.T;
#pragma unroll
            for (int ot = 0; ot < OT; ++ot)
                buffer_store4<0>(dstB, live ? oOff[ot] : kOutOfRange, uniform + hf * 64,
                                       make_float4(acc[hf][ot][0], acc[hf][ot][1], acc[hf][ot][2], acc[hf][ot][3]));
        }
    };

    {
        // Trip k loads (pair, pass) number k of the range into registers, multiplies number k - 1 from its patch and
        // then writes the registers to the other patch (or, with one patch, to the same after a barrier); the first
        // trip only loads.  Pairs are numbered with the pixel block fastest, then the step, then the batch item.
        const int perItem = static_cast<int>(g.byBlocks.d);   // pixel blocks of a batch item
        int image = static_cast<int>(fastdiv(static_cast<uint32_t>(p0), g.byBlocks));
        int inItem = p0 - image * perItem;
        int item = static_cast<int>(fastdiv(static_cast<uint32_t>(image), g.bySteps));
        int st = image - item * g.steps, pass = 0;
        int stCur = 0, passCur = 0, pixCur = -1, nCur = -1, nNext = -1;
        float4 R[NS];
        int buf = DOUBLE ? 1 : 0;
        bool first = true;
        const int trips = (p1 - p0) * g.passes;
        clear();
#pragma nounroll
        for (int k = 0;; ++k) {
            const bool more = k < trips;
            bool moved = first;
            if (more && !first) {
                if (++pass == g.passes) {
                    pass = 0;
                    moved = true;
                    if (++inItem == perItem) {
                        inItem = 0;
                        if (++st == g.steps) {
                            st = 0;
                            ++item;
                        }
                    }
                }
            }
            if (more && moved) nNext = place(item * perItem + inItem);
            issue(R, st, pass, more);
            __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the matrix work
            if (!first) {
                using I0 = std::integral_constant<int, 0>;
                using I1 = std::integral_constant<int, 1>;
                using I2 = std::integral_constant<int, 2>;
                if ((stCur << 5) + 16 < g.T) {
                    if (DOUBLE && buf != 0) multiply(I1{}, I2{}, passCur, 1);
                    else multiply(I0{}, I2{}, passCur, 0);
                } else {
                    if (DOUBLE && buf != 0) multiply(I1{}, I1{}, passCur, 1);
                    else multiply(I0{}, I1{}, passCur, 0);
                }
                if (passCur == g.passes - 1) {
                    if (nCur >= 0) {
                        dstB = make_buffer(g.dst + (static_cast<int64_t>(nCur) * g.DC + static_cast<int64_t>(grp) * g.Mg) * dstPlane);
                        store(pixCur, stCur);
                    }
                    clear();
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (!more) break;
            if (DOUBLE) buf ^= 1;
            else __syncthreads();           // every wavefront has read the one patch
            stage(R, buf);
            stCur = st; passCur = pass; pixCur = pixNext; nCur = nNext;
            __syncthreads();
            first = false;
        }
    }
}

// ---- weight gradient on the matrix cores, input patch of a block of pixels in LDS -------------------
// The kernel above fetches every input row once per tap that uses it (the working set of four
// wavefronts does not stay in the 32 KB L1), 64 bytes at a time: it is bound by the number of cache
// line requests a compute unit can have in flight.  Here a work-group takes kWgPix consecutive output
// pixels of one output row at a time and, per step of 32 time samples, copies the input patch under
// those pixels - the channels of its column group x KH filter rows x WX columns, one whole 128-byte
// line each - into LDS once (out-of-image positions as zeros); the B operands of all pixels and taps
// come from there with one 16-byte LDS read per tile and half step, the A operands (gradOut rows,
// used once) straight from global memory, both halves of a line by consecutive instructions.  The
// eight 16-byte units of a patch row are stored at (unit ^ row % 8), so that the 16 lanes of a read,
// which address 16 different rows, spread over the banks.  Two patches are resident: while the matrix
// instructions work on one, the loads of the next (pixel block, step) pair are in flight in registers
// and are written to the other before the pair's single barrier.  A work-group owns a contiguous
// range of the pairs of the whole batch, so all work-groups do the same amount of work whatever the
// map's size; each wavefront takes one pixel, and the four add their tiles up in LDS at the end, in
// wavefront order, into one workspace row per range.
constexpr int kWgPix = 4;            // pixels per block (one per wavefront)
constexpr int kWgRow = 128;          // bytes per patch row: 32 samples
constexpr int kWgMaxRows = 288;      // patch rows per buffer (9 passes of 32); row kWgMaxRows of a buffer holds zeros
constexpr int kWgBuf = (kWgMaxRows + 1) * kWgRow;

struct WgradLdsArgs {
    const float *gradOut, *in;
    float *partial;
    SynGeom s;
    int Cg, Og, CK;
    int oGroups, colGroups;
    int WX, rows;              // patch width in input pixels, patch rows = channels * KH * WX
    int blocksPerRow, steps;   // pixel blocks per output row, steps of 32 samples per row
    int pairs, slices, pairsPerSlice, nW;
    FastDiv byColGroups, byOGroups, byGroups, byKK, byKW, bySteps, byBlocks, byBlocksPerRow, byPatch, byWX;
};

template <int MT, int NT, int NS>
__global__ __launch_bounds__(256, 2) void synapse_wgrad_lds_kernel(WgradLdsArgs g)
{
    extern __shared__ __align__(16) float lds[];
    char *const ldsBytes = reinterpret_cast<char *>(lds);
    const SynGeom &s = g.s;
    uint32_t rest = xcd_contiguous(blockIdx.x, gridDim.x);
    uint32_t qq = fastdiv(rest, g.byColGroups);
    const int cg = static_cast<int>(rest - qq * g.byColGroups.d);
    rest = qq; qq = fastdiv(rest, g.byOGroups);
    const int og = static_cast<int>(rest - qq * g.byOGroups.d);
    rest = qq; qq = fastdiv(rest, g.byGroups);
    const int grp = static_cast<int>(rest - qq * g.byGroups.d);
    const int slice = static_cast<int>(qq);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, r = lane & 15, h = lane >> 4;
    const int c0 = static_cast<int>(fastdiv(static_cast<uint32_t>(cg * NT * 16), g.byKK));  // first channel of the column group
    const int64_t goPlane = static_cast<int64_t>(s.OH) * s.OW * s.T, inPlane = static_cast<int64_t>(s.H) * s.W * s.T;
    BufferRsrc goB = make_buffer(g.gradOut), inB = make_buffer(g.in);   // (of the batch item at hand: set by place())
    const int rowBytes = s.W * s.T * 4, pixBytes = s.T * 4;

    // This lane copies unit u (samples 4u..4u+3 of the step) of patch rows tid / 8 + 32 m, m < NS; a patch row is
    // (channel, filter row, patch column).  (tid / 8 + 32 m) % 8 does not depend on m: one LDS address, immediate
    // offsets for the passes.
    const int u = tid & 7;
    const int stageAddr = (tid >> 3) * kWgRow + ((u ^ ((tid >> 3) & 7)) << 4);

    // rows of this lane: output channel of every A tile, patch row (this wavefront's pixel) of every B tile
    int offA[MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
        const int o = ((og * MT + mt) << 4) + r;
        offA[mt] = masked_offset(o < g.Og, o * static_cast<int>(goPlane) * 4 + h * 16);
    }
    int bAddr[2][NT];                      // (columns past the filter read the zero row)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const int col = ((cg * NT + nt) << 4) + r;
        const uint32_t cl = fastdiv(static_cast<uint32_t>(col), g.byKK);
        const int ij = col - static_cast<int>(cl * g.byKK.d);
        const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(ij), g.byKW));
        const int j = ij - i * s.KW;
        const int row = col < g.CK ? ((static_cast<int>(cl) - c0) * s.KH + i) * g.WX + j * s.dW + wave * s.sW : kWgMaxRows;
        bAddr[0][nt] = row * kWgRow + ((h ^ (row & 7)) << 4);
        bAddr[1][nt] = row * kWgRow + (((4 + h) ^ (row & 7)) << 4);
    }

    floatx4 acc[MT][NT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) acc[mt][nt] = floatx4{0.f, 0.f, 0.f, 0.f};

    if (tid < 2 * (kWgRow / 4)) {
        const int b = tid / (kWgRow / 4), e = tid - b * (kWgRow / 4);
        lds[(b * kWgBuf + kWgMaxRows * kWgRow) / 4 + e] = 0.f;
    }

    const int p0 = slice * g.pairsPerSlice, p1 = min(g.pairs, p0 + g.pairsPerSlice);
    int sOff[NS], aOff[MT];
    // offsets of a pixel block: patch positions outside the image, or right of what the block's valid
    // pixels read, are loaded as zeros; so are the A rows of pixels past the end of the output row
    auto place = [&](int blockOfAll) {
        const int n = static_cast<int>(fastdiv(static_cast<uint32_t>(blockOfAll), g.byBlocks));
        const int block = blockOfAll - n * static_cast<int>(g.byBlocks.d);
        goB = make_buffer(g.gradOut + (static_cast<int64_t>(n) * s.O + grp * g.Og) * goPlane);
        inB = make_buffer(g.in + (static_cast<int64_t>(n) * s.C + grp * g.Cg + c0) * inPlane);
        const int a = static_cast<int>(fastdiv(static_cast<uint32_t>(block), g.byBlocksPerRow));
        const int b0 = (block - a * g.blocksPerRow) * kWgPix;
        const int nv = min(kWgPix, s.OW - b0);
        const int xLimit = (nv - 1) * s.sW + (s.KW - 1) * s.dW + 1;
        const int y0 = a * s.sH - s.pH, x0 = b0 * s.sW - s.pW;
#pragma unroll
        for (int m = 0; m < NS; ++m) {
            const int row = (tid >> 3) + 32 * m;
            const uint32_t cl = fastdiv(static_cast<uint32_t>(row), g.byPatch);
            const int rem = row - static_cast<int>(cl * g.byPatch.d);
            const int i = static_cast<int>(fastdiv(static_cast<uint32_t>(rem), g.byWX));
            const int x = rem - i * g.WX;
            const int y = y0 + i * s.dH, xx = x0 + x;
            const bool ok = row < g.rows && c0 + static_cast<int>(cl) < g.Cg && x < xLimit &&
                            static_cast<unsigned>(y) < static_cast<unsigned>(s.H) &&
                            static_cast<unsigned>(xx) < static_cast<unsigned>(s.W);
            sOff[m] = masked_offset(ok, static_cast<int>(cl) * static_cast<int>(inPlane) * 4 + y * rowBytes + xx * pixBytes + u * 16);
        }
        const int b = b0 + wave;
        const int pix = (a * s.OW + b) * pixBytes;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) aOff[mt] = masked_offset(b < s.OW && offA[mt] != kOutOfRange, offA[mt] + pix);
    };
    // Always the same number of loads, masked when there is no next pair: the waits in the loop then leave
    // exactly this batch in flight on every path.  `plain`: every sample of the step exists, so the block's
    // offsets are used as they are.
    auto issue = [&](float4 (&R)[NS], float4 (&A)[2][MT], int st, bool more) {
        const int tBytes = st << 7;
        if (more && (st << 5) + 32 <= s.T) {
#pragma unroll
            for (int m = 0; m < NS; ++m) R[m] = buffer_load4<0>(inB, sOff[m], tBytes);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                A[0][mt] = buffer_load4<0>(goB, aOff[mt], tBytes);
                A[1][mt] = buffer_load4<0>(goB, aOff[mt], tBytes + 64);
            }
        } else {
            const bool liveU = more && (st << 5) + (u << 2) < s.T;
            const bool liveH0 = more && (st << 5) + (h << 2) < s.T, liveH1 = more && (st << 5) + 16 + (h << 2) < s.T;
#pragma unroll
            for (int m = 0; m < NS; ++m) R[m] = buffer_load4<0>(inB, liveU ? sOff[m] : kOutOfRange, tBytes);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
                A[0][mt] = buffer_load4<0>(goB, liveH0 ? aOff[mt] : kOutOfRange, tBytes);
                A[1][mt] = buffer_load4<0>(goB, liveH1 ? aOff[mt] : kOutOfRange, tBytes + 64);
            }
        }
    };
    // registers -> patch; a wavefront notes whether any of its samples has more than the upper 16 bits
    uint32_t *const flags = reinterpret_cast<uint32_t *>(ldsBytes + 2 * kWgBuf);   // [2][4]
    auto stage = [&](const float4 (&R)[NS], int buf) {
        uint32_t low = 0;
#pragma unroll
        for (int m = 0; m < NS; ++m) {
            *reinterpret_cast<float4 *>(ldsBytes + buf + stageAddr + m * 32 * kWgRow) = R[m];
            low |= (__builtin_bit_cast(uint32_t, R[m].x) | __builtin_bit_cast(uint32_t, R[m].y)) |
                   (__builtin_bit_cast(uint32_t, R[m].z) | __builtin_bit_cast(uint32_t, R[m].w));
        }
        const bool any = __builtin_amdgcn_ballot_w64((low & 0xffffu) != 0u) != 0;
        if (lane == 0) flags[(buf != 0 ? 4 : 0) + wave] = any ? 1u : 0u;
    };
    // One v_mfma_f32_16x16x32_bf16 takes a tile through all 32 samples of the step: slot 8 h + e of the reduction is
    // sample 4 h + e (e < 4) or 16 + 4 h + e - 4 of the step, which is what a lane holds of a row of gradOut (two
    // 16-byte loads) and reads of a patch row (two 16-byte reads).  The rows of gradOut are split into three bf16
    // parts per number (fir_core.h); the patch rows are, too - or, when the patch holds nothing beyond the upper 16
    // bits of its numbers (spikes), only packed: three products per tile instead of six.  Samples past the end of
    // a row were loaded as zeros.
    auto multiply = [&](const float4 (&A)[2][MT], int buf) {
        const bool allParts = __builtin_amdgcn_ballot_w64(lane < 4 && flags[(buf != 0 ? 4 : 0) + (lane & 3)] != 0u) != 0;
        SplitPlanes a[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
            const float v[8] = {A[0][mt].x, A[0][mt].y, A[0][mt].z, A[0][mt].w, A[1][mt].x, A[1][mt].y, A[1][mt].z, A[1][mt].w};
            a[mt] = split_bf16(v);
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            const float4 b0 = *reinterpret_cast<const float4 *>(ldsBytes + buf + bAddr[0][nt]);
            const float4 b1 = *reinterpret_cast<const float4 *>(ldsBytes + buf + bAddr[1][nt]);
            const float v[8] = {b0.x, b0.y, b0.z, b0.w, b1.x, b1.y, b1.z, b1.w};
            if (allParts) {
                const SplitPlanes b = split_bf16(v);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[mt][nt] = mfma_bf16(a[mt].lo, b.hi, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].hi, b.lo, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].mid, b.mid, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].mid, b.hi, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].hi, b.mid, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].hi, b.hi, acc[mt][nt]);
                }
            } else {
                uint4_ext bh;
#pragma unroll
                for (int w2 = 0; w2 < 4; ++w2)
                    bh[w2] = __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, v[2 * w2 + 1]), __builtin_bit_cast(uint32_t, v[2 * w2]), 0x07060302u);
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
                    acc[mt][nt] = mfma_bf16(a[mt].lo, bh, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].mid, bh, acc[mt][nt]);
                    acc[mt][nt] = mfma_bf16(a[mt].hi, bh, acc[mt][nt]);
                }
            }
        }
    };

    {
        // Trip k of the loop loads pair p0 + k into registers, multiplies pair p0 + k - 1 from its LDS buffer
        // ((k - 1) % 2) and then writes the registers to the other buffer: the loop's code exists once, its
        // first trip only loads.
        int block = static_cast<int>(fastdiv(static_cast<uint32_t>(p0), g.bySteps));
        int st = p0 - block * g.steps;
        float4 R[NS], A[2][MT];
        int buf = kWgBuf;
        bool first = true;
#pragma nounroll
        for (int p = p0 - 1;; ++p) {
            const bool more = p + 1 < p1;
            bool moved = first;
            if (more && !first && ++st == g.steps) {
                st = 0;
                ++block;
                moved = true;
            }
            if (more && moved) place(block);
            float4 An[2][MT];
            issue(R, An, st, more);
            __builtin_amdgcn_sched_barrier(0);  // the loads stay ahead of the pair's matrix work
            if (!first) multiply(A, buf);
            __builtin_amdgcn_sched_barrier(0);
            if (!more) break;
            buf = kWgBuf - buf;
            stage(R, buf);
#pragma unroll
            for (int hf = 0; hf < 2; ++hf)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) A[hf][mt] = An[hf][mt];
            __syncthreads();
            first = false;
        }
    }

    // every wavefront puts its tiles into LDS (the patches are no longer needed); the work-group adds the four
    // copies in wavefront order and writes one workspace row.  Element v of a lane's accumulator is row 4 * h + v,
    // column r of the tile.
    __syncthreads();
    floatx4 *const red = reinterpret_cast<floatx4 *>(lds);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) red[(wave * MT * NT + mt * NT + nt) * 64 + lane] = acc[mt][nt];
    __syncthreads();
    float *row = g.partial + static_cast<int64_t>(slice) * g.nW;
#pragma unroll 1
    for (int e = tid; e < MT * NT * 64; e += 256) {
        const int tile = e >> 6, l = e & 63;
        const int mt = tile / NT, nt = tile - mt * NT;
        const floatx4 sum = ((red[e] + red[MT * NT * 64 + e]) + red[2 * MT * NT * 64 + e]) + red[3 * MT * NT * 64 + e];
        const int o = ((og * MT + mt) << 4) + ((l >> 4) << 2);
        const int col = ((cg * NT + nt) << 4) + (l & 15);
        if (col < g.CK) {
            float *cell = row + static_cast<int64_t>(grp * g.Og + o) * g.CK + col;
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (o + v < g.Og) cell[static_cast<int64_t>(v) * g.CK] = sum[v];
        }
    }
}

// gradW[q] = sum of the workspace rows: lane (q, part) adds rows part, part+PARTS, ... in order, then
// the PARTS sums of a weight are added in order (a fixed association for a given geometry).  A group
// handles 256 / PARTS weights; few weights take more parts so that the launch still fills the GPU.
template <int PARTS>
__global__ __launch_bounds__(256) void synapse_wgrad_sum_kernel(float *__restrict__ gradW,
                                                                const float *__restrict__ partial, int rows, int nW)
{
    constexpr int kWeights = 256 / PARTS;
    __shared__ float part[PARTS][kWeights + 1];
    const int ql = threadIdx.x % kWeights, pt = threadIdx.x / kWeights;
    const int q = blockIdx.x * kWeights + ql;
    float acc = 0.f;
    if (q < nW)
        for (int r = pt; r < rows; r += PARTS) acc += partial[static_cast<int64_t>(r) * nW + q];
    part[pt][ql] = acc;
    __syncthreads();
    if (threadIdx.x < kWeights && q < nW) {
        float v = part[0][ql];
#pragma unroll
        for (int k = 1; k < PARTS; ++k) v += part[k][ql];
        gradW[q] = v;
    }
}

static void launch_wgrad_sum(float *gradW, const float *workspace, int rows, int nW, hipStream_t st)
{
    if (nW < 2048)
        hipLaunchKernelGGL(synapse_wgrad_sum_kernel<64>, dim3(static_cast<unsigned>(ceil_div(nW, 4))), dim3(256), 0, st,
                           gradW, workspace, rows, nW);
    else
        hipLaunchKernelGGL(synapse_wgrad_sum_kernel<16>, dim3(static_cast<unsigned>(ceil_div(nW, 16))), dim3(256), 0, st,
                           gradW, workspace, rows, nW);
}

// ---- host side -------------------------------------------------------------------------------------
static int out_extent(int64_t in, int64_t k, int64_t s, int64_t p, int64_t d)
{
    const int64_t span = in + 2 * p - d * (k - 1) - 1;
    return span < 0 ? 0 : static_cast<int>(span / s + 1);
}

// Validates the caller's geometry and fills the derived output extents.
static int check_geom(const slayer_synapse_geom *c, SynGeom &s)
{
    if (!c) return SLAYER_EINVAL;
    s = SynGeom{c->N, c->C, c->H, c->W, c->T, c->O, c->KH, c->KW, c->strideH, c->strideW, c->padH,
                c->padW, c->dilH, c->dilW, c->groups, 0, 0};
    if (s.N < 0 || s.C < 0 || s.H < 0 || s.W < 0 || s.T < 0 || s.O < 0) return SLAYER_EINVAL;
    if (s.KH < 1 || s.KW < 1 || s.sH < 1 || s.sW < 1 || s.dH < 1 || s.dW < 1 || s.pH < 0 || s.pW < 0) return SLAYER_EINVAL;
    if (s.groups < 1 || s.C % s.groups || s.O % s.groups) return SLAYER_EINVAL;
    s.OH = out_extent(s.H, s.KH, s.sH, s.pH, s.dH);
    s.OW = out_extent(s.W, s.KW, s.sW, s.pW, s.dW);
    // the kernels index one batch item with 32-bit byte offsets, and the padded extents with int
    // (with room for the few rows by which the gather kernel's buffer starts before the tensor)
    const int64_t limit = (1LL << 31) - (1LL << 24);
    if (static_cast<int64_t>(s.C) * s.H * s.W * s.T * 4 >= limit) return SLAYER_EUNSUPPORTED;
    if (static_cast<int64_t>(s.O) * s.OH * s.OW * s.T * 4 >= limit) return SLAYER_EUNSUPPORTED;
    if (static_cast<int64_t>(s.H) + 2LL * s.pH + static_cast<int64_t>(s.dH) * s.KH >= (1 << 24)) return SLAYER_EUNSUPPORTED;
    // the taps' span in bytes, by which that buffer is moved
    if ((static_cast<int64_t>(s.pH) + static_cast<int64_t>(s.dH) * s.KH) * s.W * s.T * 4 +
            (static_cast<int64_t>(s.pW) + static_cast<int64_t>(s.dW) * s.KW) * s.T * 4 >= (1LL << 24))
        return SLAYER_EUNSUPPORTED;
    if (static_cast<int64_t>(s.W) + 2LL * s.pW + static_cast<int64_t>(s.dW) * s.KW >= (1 << 24)) return SLAYER_EUNSUPPORTED;
    if (static_cast<int64_t>(s.C / s.groups) * s.KH * s.KW >= (1 << 24)) return SLAYER_EUNSUPPORTED;
    if (static_cast<int64_t>(s.O) * (s.C / s.groups) * s.KH * s.KW >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    return SLAYER_OK;
}

template <int MB, int VEC, bool BACKWARD>
static void launch_gather_mb(const GatherArgs &g, bool strided, unsigned blocks, hipStream_t st)
{
    if (strided)
        hipLaunchKernelGGL((synapse_gather_kernel<MB, VEC, BACKWARD, true>), dim3(blocks), dim3(256), 0, st, g);
    else
        hipLaunchKernelGGL((synapse_gather_kernel<MB, VEC, BACKWARD, false>), dim3(blocks), dim3(256), 0, st, g);
}

// The matrix-core gather: unit stride in the gradient (forward: any stride), rows of whole vectors, passes of
// whole source channels that fill most of the 36 tap steps, at least 16 destination channels, patch and weights
// within LDS.  Returns SLAYER_EUNSUPPORTED (nothing launched) when the geometry does not qualify.
template <bool BACKWARD>
static int launch_gather_mfma(const GatherArgs &a, const SynGeom &s, bool strided, hipStream_t st)
{
    if (strided || a.Mg < 16) return SLAYER_EUNSUPPORTED;
    const int KK = a.KH * a.KW;
    if (KK > 4 * kGmSteps) return SLAYER_EUNSUPPORTED;
    int chans = 4 * kGmSteps / KK;
    if (chans > a.Qg) chans = a.Qg;
    if (chans < 1 || a.Qg % chans != 0 || chans * KK < 96) return SLAYER_EUNSUPPORTED;
    const int passes = a.Qg / chans;
    const int OT = (a.Mg >= 32 && passes * 2 <= 4) ? 2 : 1;
    if (passes * OT > 4) return SLAYER_EUNSUPPORTED;
    const int absStepW = a.stepW < 0 ? -a.stepW : a.stepW;
    const int64_t WX = static_cast<int64_t>(kGmPix - 1) * a.mulW + static_cast<int64_t>(a.KW - 1) * absStepW + 1;
    const int64_t rows = static_cast<int64_t>(chans) * a.KH * WX;
    if (rows > kGmMaxRows) return SLAYER_EUNSUPPORTED;
    GatherMfmaArgs g{};
    g.src = a.src; g.dst = a.dst; g.w = a.w;
    g.SC = a.SC; g.SH = a.SH; g.SW = a.SW; g.DC = a.DC; g.DH = a.DH; g.DW = a.DW; g.T = a.T;
    g.Qg = a.Qg; g.Mg = a.Mg; g.groups = a.groups; g.KH = a.KH; g.KW = a.KW; g.Cg = a.Cg; g.Og = a.Og;
    g.mulH = a.mulH; g.mulW = a.mulW; g.offH = a.offH; g.offW = a.offW; g.stepH = a.stepH; g.stepW = a.stepW;
    g.chansPerPass = chans; g.passes = passes; g.WX = static_cast<int>(WX);
    g.xBias = a.stepW < 0 ? (a.KW - 1) * absStepW : 0;
    g.rows = static_cast<int>(rows);
    g.oGroups = static_cast<int>(ceil_div(a.Mg, 16 * OT));
    g.blocksPerRow = static_cast<int>(ceil_div(a.DW, kGmPix));
    g.steps = (a.T + 31) / 32;
    const int64_t pairs = static_cast<int64_t>(s.N) * a.DH * g.blocksPerRow * g.steps;
    if (pairs < 1 || pairs >= (1LL << 30)) return SLAYER_EUNSUPPORTED;
    g.pairs = static_cast<int>(pairs);
    // one work-group per compute unit (its LDS); a few short of the 256 places
    const int64_t base = static_cast<int64_t>(a.groups) * g.oGroups;
    int64_t slices = 252 / base;
    if (slices < 1) slices = 1;
    if (slices > pairs) slices = pairs;
    g.pairsPerSlice = static_cast<int>(ceil_div(pairs, slices));
    g.slices = static_cast<int>(ceil_div(pairs, g.pairsPerSlice));
    g.byOGroups = make_fastdiv(static_cast<uint32_t>(g.oGroups));
    g.byGroups = make_fastdiv(static_cast<uint32_t>(a.groups));
    g.byKK = make_fastdiv(static_cast<uint32_t>(KK));
    g.byKW = make_fastdiv(static_cast<uint32_t>(a.KW));
    g.bySteps = make_fastdiv(static_cast<uint32_t>(g.steps));
    g.byBlocks = make_fastdiv(static_cast<uint32_t>(a.DH * g.blocksPerRow));
    g.byBlocksPerRow = make_fastdiv(static_cast<uint32_t>(g.blocksPerRow));
    g.byPatch = make_fastdiv(static_cast<uint32_t>(a.KH * g.WX));
    g.byWX = make_fastdiv(static_cast<uint32_t>(g.WX));
    const int64_t blocks = base * g.slices;
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    if constexpr (BACKWARD) {
        // The source is a gradient tensor: numbers with all their bits, which the bf16 kernel would have to split in
        // registers, tap by tap (137 us against 120 us on the 16 -> 32 channel layer): the fp32 instructions stay.
        const int ldsBytes = 2 * kGmBuf + passes * OT * 64 * kGmSteps * 4;
        // more LDS than a kernel may use without asking; asked once per device (a host-side setting, no allocation)
        static std::atomic<bool> raised[2][64];
        int device = 0;
        hipError_t err = hipGetDevice(&device);
        if (err == hipSuccess && (device < 0 || device >= 64)) err = hipErrorInvalidDevice;
        if (err == hipSuccess && !raised[OT - 1][device].load(std::memory_order_acquire)) {
            const void *fn = OT == 2 ? reinterpret_cast<const void *>(&synapse_gather_mfma_kernel<2, BACKWARD>)
                                     : reinterpret_cast<const void *>(&synapse_gather_mfma_kernel<1, BACKWARD>);
            err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kGmBuf + kGmMaxWeightBytes);
            if (err == hipSuccess) raised[OT - 1][device].store(true, std::memory_order_release);
        }
        if (err != hipSuccess) return note_hip_error(err);
        const dim3 grid(static_cast<unsigned>(blocks));
        if (OT == 2) hipLaunchKernelGGL((synapse_gather_mfma_kernel<2, BACKWARD>), grid, dim3(512), ldsBytes, st, g);
        else hipLaunchKernelGGL((synapse_gather_mfma_kernel<1, BACKWARD>), grid, dim3(512), ldsBytes, st, g);
        return launch_status();
    } else {
        const int units = passes * OT;
        const bool twoPatches = units <= 2;      // (beside the weights of two sets; more leave room for one patch)
        const int ldsBytes = (twoPatches ? 2 * kGmBuf : kGmBuf) + units * kGsUnitBytes + 64;
        // more LDS than a kernel may use without asking; asked once per device (a host-side setting, no allocation)
        static std::atomic<bool> raised[2][2][64];
        int device = 0;
        hipError_t err = hipGetDevice(&device);
        if (err == hipSuccess && (device < 0 || device >= 64)) err = hipErrorInvalidDevice;
        const void *fn = OT == 2 ? (twoPatches ? reinterpret_cast<const void *>(&synapse_gather_split_kernel<2, BACKWARD, true>)
                                               : reinterpret_cast<const void *>(&synapse_gather_split_kernel<2, BACKWARD, false>))
                                 : (twoPatches ? reinterpret_cast<const void *>(&synapse_gather_split_kernel<1, BACKWARD, true>)
                                               : reinterpret_cast<const void *>(&synapse_gather_split_kernel<1, BACKWARD, false>));
        if (err == hipSuccess && !raised[OT - 1][twoPatches][device].load(std::memory_order_acquire)) {
            err = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (twoPatches ? 2 * kGmBuf + 2 * kGsUnitBytes : kGmBuf + 4 * kGsUnitBytes) + 64);
            if (err == hipSuccess) raised[OT - 1][twoPatches][device].store(true, std::memory_order_release);
        }
        if (err != hipSuccess) return note_hip_error(err);
        const dim3 grid(static_cast<unsigned>(blocks));
        if (OT == 2) {
            if (twoPatches) hipLaunchKernelGGL((synapse_gather_split_kernel<2, BACKWARD, true>), grid, dim3(512), ldsBytes, st, g);
            else hipLaunchKernelGGL((synapse_gather_split_kernel<2, BACKWARD, false>), grid, dim3(512), ldsBytes, st, g);
        } else {
            if (twoPatches) hipLaunchKernelGGL((synapse_gather_split_kernel<1, BACKWARD, true>), grid, dim3(512), ldsBytes, st, g);
            else hipLaunchKernelGGL((synapse_gather_split_kernel<1, BACKWARD, false>), grid, dim3(512), ldsBytes, st, g);
        }
        return launch_status();
    }
}

template <bool BACKWARD>
static int launch_gather(float *dst, const float *src, const float *w, const SynGeom &s, hipStream_t st)
{
    GatherArgs g{};
    g.src = src; g.dst = dst; g.w = w;
    g.T = s.T; g.groups = s.groups; g.KH = s.KH; g.KW = s.KW;
    g.Cg = s.C / s.groups; g.Og = s.O / s.groups;
    bool strided = false;
    if (!BACKWARD) {
        g.SC = s.C; g.SH = s.H; g.SW = s.W; g.DC = s.O; g.DH = s.OH; g.DW = s.OW;
        g.Qg = g.Cg; g.Mg = g.Og;
        g.mulH = s.sH; g.mulW = s.sW; g.offH = -s.pH; g.offW = -s.pW; g.stepH = s.dH; g.stepW = s.dW;
        g.divH = make_fastdiv(1); g.divW = make_fastdiv(1);
    } else {
        g.SC = s.O; g.SH = s.OH; g.SW = s.OW; g.DC = s.C; g.DH = s.H; g.DW = s.W;
        g.Qg = g.Og; g.Mg = g.Cg;
        g.mulH = 1; g.mulW = 1; g.offH = s.pH; g.offW = s.pW; g.stepH = -s.dH; g.stepW = -s.dW;
        g.divH = make_fastdiv(static_cast<uint32_t>(s.sH)); g.divW = make_fastdiv(static_cast<uint32_t>(s.sW));
        strided = s.sH > 1 || s.sW > 1;
    }
    const int64_t dstElems = static_cast<int64_t>(s.N) * g.DC * g.DH * g.DW * g.T;
    if (dstElems == 0) return SLAYER_OK;
    const bool vec = s.T % 4 == 0 && aligned16(src) && aligned16(dst);
    const int VEC = vec ? 4 : 1;
    if (BACKWARD && s.C == 1 && s.O == 1 && s.sH == s.KH && s.sW == s.KW && s.pH == 0 && s.pW == 0 && s.dH == 1 &&
        s.dW == 1 && s.OH > 0 && s.OW > 0 && !generic_forced()) {
        WindowArgs a{};
        a.gradOut = src; a.w = w; a.gradIn = dst;
        a.H = s.H; a.W = s.W; a.OH = s.OH; a.OW = s.OW; a.T = s.T; a.KW = s.KW;
        a.P = s.H * s.W * (s.T / VEC);
        a.chunks = static_cast<int>(ceil_div(a.P, 256));
        const int64_t nBlocks = static_cast<int64_t>(s.N) * a.chunks;
        if (nBlocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
        a.byChunks = make_fastdiv(static_cast<uint32_t>(a.chunks));
        a.byTV = make_fastdiv(static_cast<uint32_t>(s.T / VEC));
        a.byW = make_fastdiv(static_cast<uint32_t>(s.W));
        a.bySH = make_fastdiv(static_cast<uint32_t>(s.sH));
        a.bySW = make_fastdiv(static_cast<uint32_t>(s.sW));
        if (vec) hipLaunchKernelGGL(synapse_window_bwd_kernel<4>, dim3(static_cast<unsigned>(nBlocks)), dim3(256), 0, st, a);
        else hipLaunchKernelGGL(synapse_window_bwd_kernel<1>, dim3(static_cast<unsigned>(nBlocks)), dim3(256), 0, st, a);
        return launch_status();
    }
    // destination channels per lane: as many as the group has, up to 16
    const int MB = g.Mg >= 12 ? 16 : g.Mg >= 6 ? 8 : g.Mg >= 3 ? 4 : g.Mg == 2 ? 2 : 1;
    if (vec && !generic_forced()) {
        const int status = launch_gather_mfma<BACKWARD>(g, s, strided, st);
        if (status != SLAYER_EUNSUPPORTED) return status;
    }
    // one or two of them, and a filter wide enough for neighbouring pixels to share source columns: PX pixels per lane
    if (MB <= 2 && vec && !strided && g.mulW == 1 && g.stepW == (BACKWARD ? -1 : 1) && (g.KW == 3 || g.KW == 5 || g.KW == 7) &&
        static_cast<int64_t>(g.Qg) * g.KH * g.KW >= 32 && !generic_forced()) {
        const int pixelGroups = static_cast<int>(ceil_div(g.DW, kGatherRowPx));
        g.P = g.DH * pixelGroups * (g.T / 4);
        g.chunks = static_cast<int>(ceil_div(g.P, 256));
        g.mBlocks = static_cast<int>(ceil_div(g.Mg, MB));
        const int64_t blocks = static_cast<int64_t>(s.N) * s.groups * g.mBlocks * g.chunks;
        if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
        g.byChunks = make_fastdiv(static_cast<uint32_t>(g.chunks));
        g.byMBlocks = make_fastdiv(static_cast<uint32_t>(g.mBlocks));
        g.byGroups = make_fastdiv(static_cast<uint32_t>(s.groups));
        g.byTV = make_fastdiv(static_cast<uint32_t>(g.T / 4));
        g.byDW = make_fastdiv(static_cast<uint32_t>(pixelGroups));
        const dim3 nb(static_cast<unsigned>(blocks));
#define SLAYER_GATHER_ROW(MBV)                                                                                          \
    do {                                                                                                                \
        if (g.KW == 3) hipLaunchKernelGGL((synapse_gather_row_kernel<MBV, 3, BACKWARD>), nb, dim3(256), 0, st, g);       \
        else if (g.KW == 5) hipLaunchKernelGGL((synapse_gather_row_kernel<MBV, 5, BACKWARD>), nb, dim3(256), 0, st, g);  \
        else hipLaunchKernelGGL((synapse_gather_row_kernel<MBV, 7, BACKWARD>), nb, dim3(256), 0, st, g);                 \
    } while (0)
        if (MB == 2) SLAYER_GATHER_ROW(2);
        else SLAYER_GATHER_ROW(1);
#undef SLAYER_GATHER_ROW
        return launch_status();
    }
    g.P = g.DH * g.DW * (g.T / VEC);
    g.chunks = static_cast<int>(ceil_div(g.P, 256));
    g.mBlocks = static_cast<int>(ceil_div(g.Mg, MB));
    const int64_t blocks = static_cast<int64_t>(s.N) * s.groups * g.mBlocks * g.chunks;
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    g.byChunks = make_fastdiv(static_cast<uint32_t>(g.chunks));
    g.byMBlocks = make_fastdiv(static_cast<uint32_t>(g.mBlocks));
    g.byGroups = make_fastdiv(static_cast<uint32_t>(s.groups));
    g.byTV = make_fastdiv(static_cast<uint32_t>(g.T / VEC));
    g.byDW = make_fastdiv(static_cast<uint32_t>(g.DW));
    const unsigned nb = static_cast<unsigned>(blocks);
#define SLAYER_GATHER(MBV)                                                        \
    do {                                                                          \
        if (vec) launch_gather_mb<MBV, 4, BACKWARD>(g, strided, nb, st);          \
        else launch_gather_mb<MBV, 1, BACKWARD>(g, strided, nb, st);              \
    } while (0)
    switch (MB) {
        case 16: SLAYER_GATHER(16); break;
        case 8: SLAYER_GATHER(8); break;
        case 4: SLAYER_GATHER(4); break;
        case 2: SLAYER_GATHER(2); break;
        default: SLAYER_GATHER(1); break;
    }
#undef SLAYER_GATHER
    return launch_status();
}

// Slices per batch item for the weight gradient: enough work-groups to fill the GPU a few times
// over, at least a few trips per lane.
struct WgradPlan {
    int OBW, TAPS, oBlocks, tapBlocks, slicesPerItem, perSlice, VEC, P;
    int64_t groupsOfWork;
};

static WgradPlan plan_wgrad(const SynGeom &s, bool vec)
{
    WgradPlan p{};
    const int KK = s.KH * s.KW, Og = s.O / s.groups, Cg = s.C / s.groups;
    p.VEC = vec ? 4 : 1;
    p.OBW = Og >= 6 ? 8 : Og >= 3 ? 4 : Og == 2 ? 2 : 1;
    p.TAPS = KK >= 7 ? 9 : KK >= 3 ? 4 : KK;  // 1, 2, 4 or 9 taps per pass
    p.oBlocks = static_cast<int>(ceil_div(Og, p.OBW));
    p.tapBlocks = static_cast<int>(ceil_div(KK, p.TAPS));
    p.P = s.OH * s.OW * (s.T / p.VEC);
    p.groupsOfWork = static_cast<int64_t>(s.N) * s.groups * p.oBlocks * Cg * p.tapBlocks;
    const int64_t want = 4096;
    int64_t slices = p.groupsOfWork > 0 ? ceil_div(want, p.groupsOfWork) : 1;
    const int64_t maxSlices = ceil_div(p.P, 256 * 4);  // keep at least four trips per lane
    if (slices > maxSlices) slices = maxSlices;
    if (slices < 1) slices = 1;
    p.perSlice = static_cast<int>(ceil_div(ceil_div(p.P, slices), 256) * 256);
    if (p.perSlice < 256) p.perSlice = 256;  // empty output: one empty slice
    p.slicesPerItem = static_cast<int>(ceil_div(p.P, p.perSlice));
    if (p.slicesPerItem < 1) p.slicesPerItem = 1;
    return p;
}


// Tiling of the matrix-core weight gradient: MT x NT tiles of 16 x 16 per wavefront (at most 18
// tiles = 72 accumulator registers), slices of pixels so that the GPU sees a few thousand wavefronts.
struct MfmaPlan {
    bool use;
    int MT, NT, oGroups, colGroups, slices, pixPerSlice;
};

static MfmaPlan plan_wgrad_mfma(const SynGeom &s)
{
    MfmaPlan p{};
    const int Og = s.O / s.groups, CK = (s.C / s.groups) * s.KH * s.KW;
    const int64_t pixels = static_cast<int64_t>(s.OH) * s.OW;
    // worth it when the 16 x 16 tiles are reasonably full and rows are whole 16-byte vectors
    p.use = s.T % 4 == 0 && s.T >= 16 && Og >= 8 && CK >= 8 && pixels > 0 && s.N > 0;
    if (!p.use) return p;
    const int oTiles = static_cast<int>(ceil_div(Og, 16)), cTiles = static_cast<int>(ceil_div(CK, 16));
    // two tiles of output channels at most: 4 x 6 tiles (one wavefront per SIMD) measured 132 us on
    // 64 channels x 288 columns, 2 x 9 tiles (two per SIMD, fewer operand loads per tile) 111 us
    p.MT = oTiles >= 2 ? 2 : 1;
    const int ntMax = 9;
    const int options[5] = {1, 2, 4, 6, 9};
    p.NT = 1;
    for (int k = 0; k < 5; ++k)
        if (options[k] <= ntMax) {
            p.NT = options[k];
            if (options[k] >= cTiles) break;
        }
    // very few tiles per wavefront mean little reuse of the operands: left to the vector kernel
    // (1 x 4 tiles on 16 channels x 50 columns: 172 us against 212 us for the vector kernel)
    if (p.MT * p.NT < 4) {
        p.use = false;
        return p;
    }
    p.oGroups = static_cast<int>(ceil_div(oTiles, p.MT));
    p.colGroups = static_cast<int>(ceil_div(cTiles, p.NT));
    const int64_t base = static_cast<int64_t>(s.N) * s.groups * p.oGroups * p.colGroups;
    // four wavefronts per work-group, one pixel each at a time: slices of a multiple of 4 pixels,
    // enough work-groups for a few per compute unit
    int64_t slices = ceil_div(1536, base);
    const int64_t quads = ceil_div(pixels, 4);
    if (slices > quads) slices = quads;
    if (slices < 1) slices = 1;
    p.pixPerSlice = static_cast<int>(ceil_div(quads, slices) * 4);
    p.slices = static_cast<int>(ceil_div(pixels, p.pixPerSlice));
    return p;
}

template <int MT>
static void launch_wgrad_mfma_nt(const WgradMfmaArgs &g, int NT, unsigned blocks, hipStream_t st)
{
    switch (NT) {
        case 9: hipLaunchKernelGGL((synapse_wgrad_mfma_kernel<MT, 9>), dim3(blocks), dim3(256), 0, st, g); break;
        case 6: hipLaunchKernelGGL((synapse_wgrad_mfma_kernel<MT, 6>), dim3(blocks), dim3(256), 0, st, g); break;
        case 4: hipLaunchKernelGGL((synapse_wgrad_mfma_kernel<MT, 4>), dim3(blocks), dim3(256), 0, st, g); break;
        case 2: hipLaunchKernelGGL((synapse_wgrad_mfma_kernel<MT, 2>), dim3(blocks), dim3(256), 0, st, g); break;
        default: hipLaunchKernelGGL((synapse_wgrad_mfma_kernel<MT, 1>), dim3(blocks), dim3(256), 0, st, g); break;
    }
}

// Returns the number of workspace rows written, or a negative status.
static int launch_wgrad_mfma(const float *gradOut, const float *in, float *workspace, const SynGeom &s,
                             const MfmaPlan &p, int nW, hipStream_t st)
{
    WgradMfmaArgs g{};
    g.gradOut = gradOut; g.in = in; g.partial = workspace; g.s = s;
    g.Cg = s.C / s.groups; g.Og = s.O / s.groups; g.CK = g.Cg * s.KH * s.KW;
    g.oGroups = p.oGroups; g.colGroups = p.colGroups; g.slices = p.slices; g.pixPerSlice = p.pixPerSlice;
    g.nW = nW;
    g.bySlices = make_fastdiv(static_cast<uint32_t>(p.slices));
    g.byColGroups = make_fastdiv(static_cast<uint32_t>(p.colGroups));
    g.byOGroups = make_fastdiv(static_cast<uint32_t>(p.oGroups));
    g.byGroups = make_fastdiv(static_cast<uint32_t>(s.groups));
    g.byKK = make_fastdiv(static_cast<uint32_t>(s.KH * s.KW));
    g.byKW = make_fastdiv(static_cast<uint32_t>(s.KW));
    g.byOW = make_fastdiv(static_cast<uint32_t>(s.OW));
    const int64_t blocks = static_cast<int64_t>(s.N) * s.groups * p.oGroups * p.colGroups * p.slices;
    if (blocks >= (1LL << 31)) return -SLAYER_EUNSUPPORTED;
    const unsigned nb = static_cast<unsigned>(blocks);
    if (p.MT == 2) launch_wgrad_mfma_nt<2>(g, p.NT, nb, st);
    else launch_wgrad_mfma_nt<1>(g, p.NT, nb, st);
    const int status = launch_status();
    return status == SLAYER_OK ? s.N * p.slices : -status;
}

// Tiling of the LDS-staged matrix-core weight gradient: the tiles of plan_wgrad_mfma, blocks of kWgPix
// pixels, and ranges of (block, step) pairs so that one wave of work-groups (two per compute unit of the
// 256) covers the tensor.
struct LdsPlan {
    bool use;
    int NS, WX, rows, blocksPerRow, steps, pairs, slices, pairsPerSlice;
};

static LdsPlan plan_wgrad_lds(const SynGeom &s, const MfmaPlan &m)
{
    LdsPlan p{};
    if (!m.use) return p;
    const int Cg = s.C / s.groups, KK = s.KH * s.KW, CK = Cg * KK;
    const int64_t WX = static_cast<int64_t>(kWgPix - 1) * s.sW + static_cast<int64_t>(s.KW - 1) * s.dW + 1;
    int channels = 0;  // most channels that one column group's columns belong to
    for (int cg = 0; cg < m.colGroups; ++cg) {
        const int col0 = cg * m.NT * 16, col1 = (CK < col0 + m.NT * 16 ? CK : col0 + m.NT * 16) - 1;
        if (col1 >= col0 && col1 / KK - col0 / KK + 1 > channels) channels = col1 / KK - col0 / KK + 1;
    }
    const int64_t rows = channels * s.KH * WX;
    if (rows < 1 || rows > kWgMaxRows) return p;
    p.use = true;
    p.WX = static_cast<int>(WX);
    p.rows = static_cast<int>(rows);
    p.NS = rows <= 96 ? 3 : rows <= 192 ? 6 : 9;       // passes of 32 rows
    p.blocksPerRow = static_cast<int>(ceil_div(s.OW, kWgPix));
    p.steps = (s.T + 31) / 32;
    const int64_t pairs = static_cast<int64_t>(s.N) * s.OH * p.blocksPerRow * p.steps;   // of the whole batch
    if (pairs >= (1LL << 30)) {
        p.use = false;
        return p;
    }
    p.pairs = static_cast<int>(pairs);
    const int64_t base = static_cast<int64_t>(s.groups) * m.oGroups * m.colGroups;
    // two work-groups per compute unit; a few short of the 512 places, which measured faster than all of them
    // (504: 110 us, 512: 123 us on the 2 -> 16 channel 5 x 5 layer)
    int64_t slices = 504 / base;
    if (slices < 1) slices = 1;
    if (slices > pairs) slices = pairs;
    p.pairsPerSlice = static_cast<int>(ceil_div(pairs, slices));
    p.slices = static_cast<int>(ceil_div(pairs, p.pairsPerSlice));
    return p;
}

template <int MT, int NT, int NS>
static int launch_wgrad_lds_one(const WgradLdsArgs &g, unsigned blocks, hipStream_t st)
{
    // two patches of kWgBuf bytes: more than the 64 KB a kernel may use without asking; asked once per device
    // (a host-side setting of the kernel, no allocation)
    static std::atomic<bool> raised[64];
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err == hipSuccess && (device < 0 || device >= 64)) err = hipErrorInvalidDevice;
    if (err == hipSuccess && !raised[device].load(std::memory_order_acquire)) {
        err = hipFuncSetAttribute(reinterpret_cast<const void *>(&synapse_wgrad_lds_kernel<MT, NT, NS>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, 2 * kWgBuf + 32);
        if (err == hipSuccess) raised[device].store(true, std::memory_order_release);
    }
    if (err != hipSuccess) return note_hip_error(err);
    hipLaunchKernelGGL((synapse_wgrad_lds_kernel<MT, NT, NS>), dim3(blocks), dim3(256), 2 * kWgBuf + 32, st, g);
    return launch_status();
}

template <int MT, int NS>
static int launch_wgrad_lds_nt(const WgradLdsArgs &g, int NT, unsigned blocks, hipStream_t st)
{
    switch (NT) {
        case 9: return launch_wgrad_lds_one<MT, 9, NS>(g, blocks, st);
        case 6: return launch_wgrad_lds_one<MT, 6, NS>(g, blocks, st);
        case 4: return launch_wgrad_lds_one<MT, 4, NS>(g, blocks, st);
        case 2: return launch_wgrad_lds_one<MT, 2, NS>(g, blocks, st);
        default: return launch_wgrad_lds_one<MT, 1, NS>(g, blocks, st);
    }
}

// Returns the number of workspace rows written, or a negative status.
static int launch_wgrad_lds(const float *gradOut, const float *in, float *workspace, const SynGeom &s,
                            const MfmaPlan &m, const LdsPlan &p, int nW, hipStream_t st)
{
    WgradLdsArgs g{};
    g.gradOut = gradOut; g.in = in; g.partial = workspace; g.s = s;
    g.Cg = s.C / s.groups; g.Og = s.O / s.groups; g.CK = g.Cg * s.KH * s.KW;
    g.oGroups = m.oGroups; g.colGroups = m.colGroups;
    g.WX = p.WX; g.rows = p.rows; g.blocksPerRow = p.blocksPerRow; g.steps = p.steps;
    g.pairs = p.pairs; g.slices = p.slices; g.pairsPerSlice = p.pairsPerSlice; g.nW = nW;
    g.byColGroups = make_fastdiv(static_cast<uint32_t>(m.colGroups));
    g.byOGroups = make_fastdiv(static_cast<uint32_t>(m.oGroups));
    g.byGroups = make_fastdiv(static_cast<uint32_t>(s.groups));
    g.byKK = make_fastdiv(static_cast<uint32_t>(s.KH * s.KW));
    g.byKW = make_fastdiv(static_cast<uint32_t>(s.KW));
    g.byBlocks = make_fastdiv(static_cast<uint32_t>(s.OH * p.blocksPerRow));
    g.bySteps = make_fastdiv(static_cast<uint32_t>(p.steps));
    g.byBlocksPerRow = make_fastdiv(static_cast<uint32_t>(p.blocksPerRow));
    g.byPatch = make_fastdiv(static_cast<uint32_t>(s.KH * p.WX));
    g.byWX = make_fastdiv(static_cast<uint32_t>(p.WX));
    const int64_t blocks = static_cast<int64_t>(s.groups) * m.oGroups * m.colGroups * p.slices;
    if (blocks >= (1LL << 31)) return -SLAYER_EUNSUPPORTED;
    const unsigned nb = static_cast<unsigned>(blocks);
    int status;
    if (m.MT == 2) {
        status = p.NS == 9 ? launch_wgrad_lds_nt<2, 9>(g, m.NT, nb, st)
               : p.NS == 6 ? launch_wgrad_lds_nt<2, 6>(g, m.NT, nb, st) : launch_wgrad_lds_nt<2, 3>(g, m.NT, nb, st);
    } else {
        status = p.NS == 9 ? launch_wgrad_lds_nt<1, 9>(g, m.NT, nb, st)
               : p.NS == 6 ? launch_wgrad_lds_nt<1, 6>(g, m.NT, nb, st) : launch_wgrad_lds_nt<1, 3>(g, m.NT, nb, st);
    }
    return status == SLAYER_OK ? p.slices : -status;
}

template <int OBW, int TAPS>
static void launch_wgrad_vec(const WgradArgs &g, int VEC, unsigned blocks, hipStream_t st)
{
    if (VEC == 4) hipLaunchKernelGGL((synapse_wgrad_kernel<OBW, TAPS, 4>), dim3(blocks), dim3(256), 0, st, g);
    else hipLaunchKernelGGL((synapse_wgrad_kernel<OBW, TAPS, 1>), dim3(blocks), dim3(256), 0, st, g);
}

template <int OBW>
static void launch_wgrad_taps(const WgradArgs &g, const WgradPlan &p, unsigned blocks, hipStream_t st)
{
    switch (p.TAPS) {
        case 9: launch_wgrad_vec<OBW, 9>(g, p.VEC, blocks, st); break;
        case 4: launch_wgrad_vec<OBW, 4>(g, p.VEC, blocks, st); break;
        case 2: launch_wgrad_vec<OBW, 2>(g, p.VEC, blocks, st); break;
        default: launch_wgrad_vec<OBW, 1>(g, p.VEC, blocks, st); break;
    }
}

}  // namespace slayer

extern "C" int slayer_synapse_out_shape(const slayer_synapse_geom *geom, int32_t *OH, int32_t *OW)
{
    slayer::SynGeom s;
    const int status = slayer::check_geom(geom, s);
    if (status != SLAYER_OK) return status;
    if (OH) *OH = s.OH;
    if (OW) *OW = s.OW;
    return SLAYER_OK;
}

extern "C" int slayer_synapse_conv_f32(float *out, const float *in, const float *weight,
                                       const slayer_synapse_geom *geom, void *stream)
{
    using namespace slayer;
    SynGeom s;
    const int status = check_geom(geom, s);
    if (status != SLAYER_OK) return status;
    const int64_t outElems = static_cast<int64_t>(s.N) * s.O * s.OH * s.OW * s.T;
    if (outElems == 0) return SLAYER_OK;
    if (!out || !in || !weight) return SLAYER_EINVAL;
    return launch_gather<false>(out, in, weight, s, static_cast<hipStream_t>(stream));
}

extern "C" int slayer_synapse_conv_grad_input_f32(float *gradIn, const float *gradOut, const float *weight,
                                                  const slayer_synapse_geom *geom, void *stream)
{
    using namespace slayer;
    SynGeom s;
    const int status = check_geom(geom, s);
    if (status != SLAYER_OK) return status;
    const int64_t inElems = static_cast<int64_t>(s.N) * s.C * s.H * s.W * s.T;
    if (inElems == 0) return SLAYER_OK;
    if (!gradIn || !weight) return SLAYER_EINVAL;
    const int64_t outElems = static_cast<int64_t>(s.N) * s.O * s.OH * s.OW * s.T;
    if (outElems > 0 && !gradOut) return SLAYER_EINVAL;
    // with an empty gradOut every tap is out of range and the kernel writes zeros
    return launch_gather<true>(gradIn, gradOut ? gradOut : gradIn, weight, s, static_cast<hipStream_t>(stream));
}

extern "C" int64_t slayer_synapse_conv_grad_weight_workspace_bytes(const slayer_synapse_geom *geom)
{
    using namespace slayer;
    SynGeom s;
    if (check_geom(geom, s) != SLAYER_OK) return 0;
    const int64_t nW = static_cast<int64_t>(s.O) * (s.C / s.groups) * s.KH * s.KW;
    if (nW == 0 || s.N == 0) return 0;
    const WgradPlan p = plan_wgrad(s, s.T % 4 == 0);
    const MfmaPlan m = plan_wgrad_mfma(s);
    const LdsPlan l = plan_wgrad_lds(s, m);
    int64_t most = p.slicesPerItem;
    if (m.use && m.slices > most) most = m.slices;
    int64_t rows = static_cast<int64_t>(s.N) * most;
    if (l.use && l.slices > rows) rows = l.slices;
    return rows * nW * static_cast<int64_t>(sizeof(float));
}

extern "C" int slayer_synapse_conv_grad_weight_f32(float *gradW, const float *gradOut, const float *in,
                                                   float *workspace, const slayer_synapse_geom *geom,
                                                   void *stream)
{
    using namespace slayer;
    SynGeom s;
    const int status = check_geom(geom, s);
    if (status != SLAYER_OK) return status;
    const int64_t nW64 = static_cast<int64_t>(s.O) * (s.C / s.groups) * s.KH * s.KW;
    if (nW64 == 0) return SLAYER_OK;
    if (!gradW) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int nW = static_cast<int>(nW64);
    const int64_t outElems = static_cast<int64_t>(s.N) * s.O * s.OH * s.OW * s.T;
    int rows = 0;
    if (outElems > 0) {
        if (!gradOut || !in || !workspace) return SLAYER_EINVAL;
        // the slicing must match slayer_synapse_conv_grad_weight_workspace_bytes: vectors only
        // when T allows them AND the pointers are aligned, otherwise the same slices of samples
        const bool vecT = s.T % 4 == 0;
        WgradPlan p = plan_wgrad(s, vecT);
        const bool vec = vecT && aligned16(gradOut) && aligned16(in);
        const MfmaPlan m = plan_wgrad_mfma(s);
        if (m.use && vec && !generic_forced()) {
            const LdsPlan l = plan_wgrad_lds(s, m);
            rows = l.use ? launch_wgrad_lds(gradOut, in, workspace, s, m, l, nW, st)
                         : launch_wgrad_mfma(gradOut, in, workspace, s, m, nW, st);
            if (rows < 0) return -rows;
            launch_wgrad_sum(gradW, workspace, rows, nW, st);
            return launch_status();
        }
        WgradArgs g{};
        g.gradOut = gradOut; g.in = in; g.partial = workspace; g.s = s;
        g.Cg = s.C / s.groups; g.Og = s.O / s.groups;
        g.oBlocks = p.oBlocks; g.tapBlocks = p.tapBlocks; g.slicesPerItem = p.slicesPerItem;
        g.nW = nW;
        if (vec) {
            g.P = p.P; g.perSlice = p.perSlice;
        } else {
            // same number of slices, four times the positions when T would have allowed vectors
            const int scale = vecT ? 4 : 1;
            p.VEC = 1;
            g.P = p.P * scale; g.perSlice = p.perSlice * scale;
        }
        g.bySlices = make_fastdiv(static_cast<uint32_t>(p.slicesPerItem));
        g.byTapBlocks = make_fastdiv(static_cast<uint32_t>(p.tapBlocks));
        g.byCg = make_fastdiv(static_cast<uint32_t>(g.Cg));
        g.byOBlocks = make_fastdiv(static_cast<uint32_t>(p.oBlocks));
        g.byGroups = make_fastdiv(static_cast<uint32_t>(s.groups));
        g.byTV = make_fastdiv(static_cast<uint32_t>(s.T / p.VEC));
        g.byOW = make_fastdiv(static_cast<uint32_t>(s.OW));
        const int64_t blocks = p.groupsOfWork * p.slicesPerItem;
        if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
        const unsigned nb = static_cast<unsigned>(blocks);
        switch (p.OBW) {
            case 8: launch_wgrad_taps<8>(g, p, nb, st); break;
            case 4: launch_wgrad_taps<4>(g, p, nb, st); break;
            case 2: launch_wgrad_taps<2>(g, p, nb, st); break;
            default: launch_wgrad_taps<1>(g, p, nb, st); break;
        }
        const int st1 = launch_status();
        if (st1 != SLAYER_OK) return st1;
        rows = s.N * p.slicesPerItem;
    }
    launch_wgrad_sum(gradW, workspace, rows, nW, st);
    return launch_status();
}

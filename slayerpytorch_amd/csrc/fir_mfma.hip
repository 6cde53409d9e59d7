// Temporal FIR of neuron rows on the matrix cores, for dense input and filters of 34 to 129 taps, where the
// register-window kernels of fir.hip are bound by FMA issue (an FIR of 77 taps needs 154 flop per 8 bytes).
// Correlation only (plain, or with the spike function's surrogate gradient applied to the samples on their way
// into LDS): the convolution's input is mostly spike trains, which the tiled kernel of fir.hip serves through
// its event-driven path.
//
// For Y[m] = sum_t X[m+t] * filt[t], the 16 outputs of block b (16 samples) of 16 rows are the 16x16 product
//
//     Y[16b + i][row c] = sum_k  filt[k - i] * X[16b + k][row c]        (k over the 15 + F samples from 16b on)
//
// of a banded Toeplitz matrix made of the filter (zero where k - i is not a tap) and the rows' samples.
//
// A work-group is ONE wavefront that walks over tiles of 16 consecutive rows.  It copies a tile into LDS with
// 16-byte loads that run through the rows' memory front to back, walks the blocks - the window of samples lives in
// registers and moves on by what one step consumes, so each step reads only the new samples from LDS (the walk is
// unrolled by the window size) - writes every output block over input that has left the window, and copies the rows
// back out the way they came in.  The next tile's samples are on their way into registers during the walk.  No
// barriers: the wavefronts of a compute unit overlap each other's memory and matrix work.
//
// Two kernels.  fir_mfma_split_kernel: tiles of 16 whole rows kept in LDS exactly as they lie in memory, for rows
// whose length spreads them over the LDS banks as it is (T / 4 odd); the product runs on bf16 instructions over a
// three-way split of both operands.  fir_mfma_kernel: every other row length (padded rows, or tiles of the time axis
// with halo), fp32 instructions, plain correlation only.
//
// The matrix instructions sum their products in their own order, so results agree with the sequential chain to
// rounding (a few 1e-7 of sum |x| |filt|), not bit for bit.  A structural zero times a non-finite sample would
// be NaN where the chain has no such term: a wavefront that meets a non-finite sample computes its outputs with the
// sequential chain over the valid taps instead.
#include "common.h"
#include "fir_core.h"

namespace slayer {

constexpr int kMfmaLdsBytes = 160 * 1024 / 8;  // per wavefront: 8 of them on a compute unit

struct MfmaFirArgs {
    float *out;
    const float *in, *filt;
    int64_t rows;
    int T, F;
    int nb;         // output blocks per tile of the time axis
    int timeTiles;  // tiles per row
    int pitch;      // floats per row in LDS; pitch / 4 is odd, which spreads the 16 rows over the banks
    int nv;         // 16-byte vectors per lane and tile that are in use (<= NV; whole rows: nv KiB of LDS)
    uint32_t nItems;
    float Ts;
    FirGate gate;  // GATED (whole rows only): the samples are in * gain * exp(-|u - theta| / tau), applied on the way into LDS
};

// ---- fp32 instructions, rows padded in LDS or cut into time tiles ------------------------------------------------
// v_mfma_f32_16x16x4_f32 takes 4 of the k per instruction: a lane (c = lane % 16, h = lane / 16) supplies
// X[.. + 4h + v] of row c for instruction v = 0..3, which are the four components of ONE 16-byte LDS read, and
// filt[16d + 4h + v - i] for i = lane % 16 and each of the D = F/16 + 1..2 blocks of the window, which it keeps in
// 4 D registers.  Its accumulator then holds outputs 4h..4h+3 of row c.
// NV: 16-byte vectors per lane and tile, NV * 64 >= 16 rows * (staged blocks * 4)
template <int D, int NV>
__global__ __launch_bounds__(64, 2) void fir_mfma_kernel(MfmaFirArgs p)
{
    extern __shared__ __align__(16) float X[];
    constexpr int W = D + 1;  // window slots: the D blocks of a tile and the block the next tile adds
    const int lane = threadIdx.x;
    const int c = lane & 15, h = lane >> 4;
    const int T = p.T, F = p.F, P = p.pitch;
    const int nBlk = (T + 15) >> 4;
    const int nInMax = p.nb + (p.timeTiles > 1 ? D - 1 : 0);  // staged blocks per row
    const int lenIn = 4 * nInMax, lenOut = 4 * p.nb;          // 16-byte vectors per row coming in / going out

    // the lane's column of the Toeplitz factor; the range check of a buffer that ends with the filter turns
    // every index that is not a tap into a zero
    const BufferRsrc bufF = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.filt), 0, F * 4, 0x00020000);
    float a[D][4];
#pragma unroll
    for (int d = 0; d < D; ++d)
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int tap = 16 * d + 4 * h + v - c;
            a[d][v] = __builtin_bit_cast(
                float, __builtin_amdgcn_raw_buffer_load_b32(bufF, masked_offset(tap >= 0 && tap < F, tap * 4), 0, 0));
        }

    struct Tile {
        int64_t row0;
        int nRows, t0, nb, nIn;
    };
    auto tile_of = [&](uint32_t i) {
        // tiles that share halo blocks (time tiles of the same rows) and memory lines (neighbouring rows) run on
        // the same die (the grid is a multiple of 8 wavefronts)
        const uint32_t item = xcd_contiguous(i, p.nItems);
        const uint32_t rowGroup = item / static_cast<uint32_t>(p.timeTiles);
        const int timeTile = static_cast<int>(item - rowGroup * static_cast<uint32_t>(p.timeTiles));
        Tile q;
        q.row0 = static_cast<int64_t>(rowGroup) * 16;
        q.nRows = static_cast<int>(min(static_cast<int64_t>(16), p.rows - q.row0));
        const int b0 = timeTile * p.nb;
        q.t0 = 16 * b0;
        q.nb = min(p.nb, nBlk - b0);
        q.nIn = min(nInMax, nBlk - b0);
        return q;
    };
    // vector e = lane + 64 k of a tile is vector e % lenIn of row e / lenIn; samples outside the row read as zeros
    float4 pre[NV];
    // the lane index behind a barrier for the optimiser: the (row, vector) sequences below do not depend on the
    // tile, and kept across the walk they would cost 2 registers per vector
    auto lane_again = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    // (a fixed number of loads and stores per tile, masked where a tile is short: the wait for a tile's loads can
    // then leave exactly the younger stores of the tile before in flight)
    auto fetch = [&](const Tile &q) {
        const BufferRsrc bufIn = make_buffer(p.in + q.row0 * T);
        RowCol rc;
        rc.init(lane_again(), lenIn, 1.0f / static_cast<float>(lenIn));
        const int dr = kWave / lenIn, dc = kWave % lenIn;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int t = q.t0 + (rc.c << 2);
            pre[k] = buffer_load4(bufIn, masked_offset(rc.r < q.nRows && t < T, (rc.r * T + t) * 4), 0);
            rc.advance(dr, dc, lenIn);
        }
    };
    auto stage = [&]() {  // the fetched vectors into LDS; true if a sample is not finite
        bool bad = false;
        RowCol rc;
        rc.init(lane_again(), lenIn, 1.0f / static_cast<float>(lenIn));
        const int dr = kWave / lenIn, dc = kWave % lenIn;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const float4 x = pre[k];
            // infinite or NaN (or four samples that add up to more than fp32 holds, which only costs time)
            bad |= ((x.x + x.y) + (x.z + x.w)) * 0.0f != 0.0f;
            if (rc.r < 16) *reinterpret_cast<float4 *>(X + rc.r * P + (rc.c << 2)) = x;
            rc.advance(dr, dc, lenIn);
        }
        return __builtin_amdgcn_ballot_w64(bad) != 0;
    };

    // 64 bytes of zeros behind the 16 rows
    const int zeroOff = 16 * P;
    if (lane < 4) *reinterpret_cast<float4 *>(X + zeroOff + 4 * lane) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

    uint32_t i = blockIdx.x;
    if (i >= p.nItems) return;
    Tile cur = tile_of(i);
    fetch(cur);
    {
        // stores that the range check drops, as many as a tile's: the first trip then finds the same instructions in
        // flight as the later ones - a tile's loads, then the stores of the tile before - so that one count serves all
        const BufferRsrc none = make_buffer(p.out, 0);
#pragma unroll
        for (int k = 0; k < NV; ++k) buffer_store4(none, (lane + kWave * k) * 16, 0, make_float4(static_cast<float>(k), 0.0f, 0.0f, 0.0f));
    }
    for (;;) {
        const bool chains = stage();
        wave_sync();
        const uint32_t iNext = i + gridDim.x;
        const bool more = iNext < p.nItems;
        // (the next tile's loads behind every wait of stage(): moved up between them, as the compiler likes to do to
        // reuse the registers one by one, each of those waits would also wait for the stores of the tile before)
        // (behind the last tile: a tile without rows, whose loads are all masked)
        Tile next = tile_of(more ? iNext : i);
        if (!more) next.nRows = 0;
        fetch(next);
        if (chains) {
            // a non-finite sample: the tile's outputs as sequential chains over the valid taps
            const int width = min(16 * cur.nb, T - cur.t0);
            for (int e = lane; e < cur.nRows * width; e += kWave) {
                const int r = e / width, t = cur.t0 + (e - r * width);
                const float *x = p.in + (cur.row0 + r) * T;
                const int taps = min(T - t, F);
                float acc = 0.0f;
                for (int k = 0; k < taps; ++k) acc = __builtin_fmaf(x[t + k], p.filt[k], acc);
                p.out[(cur.row0 + r) * T + t] = acc * p.Ts;
            }
        } else {
            // walk: step j makes output block j from input blocks j .. j + D - 1 and writes it over input block j
            float *col = X + c * P + 4 * h;
            const float *zeros = X + zeroOff + 4 * h;
            const int nIn = cur.nIn;
            // block q of the lane's row; behind the row, 16 bytes of zeros (choosing the address instead of masking
            // the data leaves nothing to do when the read returns, so it can stay in flight during the step)
            auto block = [&](int q) { return *reinterpret_cast<const float4 *>(q < nIn ? col + 16 * q : zeros); };
            float4 w[W];
#pragma unroll
            for (int d = 0; d < D; ++d) w[d] = block(d);
            for (int j0 = 0; j0 < cur.nb; j0 += W) {
#pragma unroll
                for (int u = 0; u < W; ++u) {
                    const int j = j0 + u;
                    if (j < cur.nb) {
                        w[(u + D) % W] = block(j + D);  // the block the next step adds
                        __builtin_amdgcn_sched_barrier(0);  // (issued here, not after the step's matrix work)
                        f32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
                        for (int d = 0; d < D; ++d) {
                            const float4 &x = w[(u + d) % W];
                            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][0], x.x, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][1], x.y, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][2], x.z, acc, 0, 0, 0);
                            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[d][3], x.w, acc, 0, 0, 0);
                        }
                        *reinterpret_cast<float4 *>(col + 16 * j) =
                            make_float4(acc.x * p.Ts, acc.y * p.Ts, acc.z * p.Ts, acc.w * p.Ts);
                    }
                }
            }
        }
        wave_sync();
        // rows back out
        const BufferRsrc bufOut = make_buffer(p.out + cur.row0 * T);
        RowCol rc;
        rc.init(lane_again(), lenOut, 1.0f / static_cast<float>(lenOut));
        const int dr = kWave / lenOut, dc = kWave % lenOut;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int t = cur.t0 + (rc.c << 2);
            const bool on = !chains && rc.r < cur.nRows && rc.c < 4 * cur.nb && t < T;
            const float4 y = *reinterpret_cast<const float4 *>(X + min(rc.r, 15) * P + (rc.c << 2));
            buffer_store4(bufOut, masked_offset(on, (rc.r * T + t) * 4), 0, y);
            rc.advance(dr, dc, lenOut);
            if (k % 8 == 7) __builtin_amdgcn_sched_barrier(0);  // a few vectors at a time: they occupy registers
        }
        if (!more) break;
        wave_sync();
        i = iNext;
        cur = next;
    }
}

// ---- the same product from bf16 instructions on a three-way split of both operands -------------------------------
// v_mfma_f32_16x16x32_bf16 multiplies 8 pairs in the time the fp32 instruction takes for one.  An fp32 number is,
// to 2^-24 of its size, the sum of three bf16 numbers: its upper 16 bits, the upper 16 bits of what is left, and
// the same again (8 + 8 + 8 significant bits, each cut, not rounded, so that all three have the number's sign and no
// part overflows).  A product of two split numbers is then the sum of nine bf16 products, each exact in the
// instruction's fp32 accumulator.  The three smallest (mid x low, low x mid, low x low: each below 2^-23 of the
// product) are left out; the six others take 6 / 8 of an fp32 instruction's time.  Measured against the exact sum,
// the result stays within 5e-7 * sum |x| |filt| (the instructions round their accumulator too) on samples and taps
// of ordinary size.  The instruction reads a bf16 operand below 2^-126 as zero, which drops parts of samples and taps
// below 2^-102 of size: at most 2^-124 * (sum |filt| + sum |x| over an output's window) in absolute terms.
// A tap that is not finite has no split, so then all tiles take the chains (as a tile with such a sample does).
//
// The rows are cut into chunks of 32 samples.  A lane (c = lane % 16, h = lane / 16) holds samples 8h .. 8h + 7 of
// each chunk of row c in the window - split once per sample, three register quadruples per chunk - and, for either
// 16-output block of a chunk, filt[32 s + 8h + e - c (- 16 for the second block)] for the window's chunks s, split the
// same way when the kernel starts.  One step makes both blocks of a chunk from the NC chunks from it on.
//
// The tile: vector e of the 16 rows' memory is vector e of LDS, no index arithmetic; the range check of the buffers
// masks what lies behind the last row of the tensor.  The last chunk of a row ends in the first samples of the next
// row, which the walk masks.
// NC: chunks in the window (the second block of a chunk reaches 31 + F samples from the chunk's start); NCE: chunks
// that the first block reaches.  NV: 16-byte vectors per lane and tile.
template <int NCE, int NC, int NV, bool GATED>
__global__ __launch_bounds__(64, 2) void fir_mfma_split_kernel(MfmaFirArgs p)
{
    extern __shared__ __align__(16) float X[];
    const int lane = threadIdx.x;
    const int c = lane & 15, h = lane >> 4;
    const int T = p.T, F = p.F;
    const int nCh = (T + 31) >> 5;

    const BufferRsrc bufF = __builtin_amdgcn_make_buffer_rsrc(const_cast<float *>(p.filt), 0, F * 4, 0x00020000);
    SplitPlanes aE[NCE], aO[NC];
    bool badTap = false;
#pragma unroll
    for (int s = 0; s < NC; ++s) {
        float fe[8], fo[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int tap = 32 * s + 8 * h + e - c;
            fe[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bufF, masked_offset(tap >= 0 && tap < F, tap * 4), 0, 0));
            fo[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bufF, masked_offset(tap >= 16 && tap - 16 < F, (tap - 16) * 4), 0, 0));
            badTap |= fe[e] * 0.0f != 0.0f || fo[e] * 0.0f != 0.0f;
        }
        if (s < NCE) aE[s] = split_bf16(fe);
        aO[s] = split_bf16(fo);
    }
    // (a tap that is not finite has no split: every tile as chains)
    const bool chainsAlways = __builtin_amdgcn_ballot_w64(badTap) != 0;

    struct Tile {
        int64_t row0;
        int nRows;
    };
    auto tile_of = [&](uint32_t i) {
        Tile q;
        q.row0 = static_cast<int64_t>(xcd_contiguous(i, p.nItems)) * 16;
        q.nRows = static_cast<int>(min(static_cast<int64_t>(16), p.rows - q.row0));
        return q;
    };
    // A tile's vectors (and, GATED, those of its potentials) come in three parts.  The first travels while the tile
    // before is walked: as many vectors as the registers hold beside the walk's operands (12 registers per chunk of
    // either filter operand and of the window; about 50 others).  The second is fetched when that walk has ended and
    // its window is free, ahead of the stores.  What does not fit beside the filter operands even then is fetched by
    // stage(), one vector for each one that it has put into LDS.
    constexpr int kRoom = (242 - 50 - 12 * (NCE + 2 * NC)) / 4;
    constexpr int kStageRoom = (242 - 50 - 12 * (NCE + NC)) / 4;
    constexpr int kAhead = (GATED ? kStageRoom / 2 : kStageRoom) < NV ? (GATED ? kStageRoom / 2 : kStageRoom) : NV;
    constexpr int kEarly = (GATED ? (kRoom + 1) / 2 : kRoom) < kAhead ? (GATED ? (kRoom + 1) / 2 : kRoom) : kAhead;
    constexpr int kEarlyU = kRoom / 2 < kAhead ? kRoom / 2 : kAhead;
    static_assert(kRoom >= 2 && kAhead >= 1, "no registers left for the tile");
    float4 pre[NV], preU[GATED ? NV : 1];
    auto fetch_one = [&](const Tile &q, int k) {
        const BufferRsrc bufIn = make_buffer(p.in + q.row0 * T, q.nRows * T * 4);
        pre[k] = buffer_load4(bufIn, lane * 16, kWave * 16 * k);
        if (GATED) {
            const BufferRsrc bufU = make_buffer(p.gate.u + q.row0 * T, q.nRows * T * 4);
            preU[k] = buffer_load4(bufU, lane * 16, kWave * 16 * k);
        }
    };
    auto fetch = [&](const Tile &q, bool second) {
        const BufferRsrc bufIn = make_buffer(p.in + q.row0 * T, q.nRows * T * 4);
        const BufferRsrc bufU = make_buffer(GATED ? p.gate.u + q.row0 * T : p.in, q.nRows * T * 4);
#pragma unroll
        for (int k = 0; k < kAhead; ++k) {
            if ((k >= kEarly) == second) pre[k] = buffer_load4(bufIn, lane * 16, kWave * 16 * k);
            if (GATED && (k >= kEarlyU) == second) preU[k] = buffer_load4(bufU, lane * 16, kWave * 16 * k);
        }
    };
    auto stage = [&](const Tile &q) {
        bool bad = false;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            float4 x = pre[k];
            if (GATED)
                x = make_float4(x.x * spike_pdf(preU[k].x, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.y * spike_pdf(preU[k].y, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.z * spike_pdf(preU[k].z, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.w * spike_pdf(preU[k].w, p.gate.theta, p.gate.tau, p.gate.gain));
            if (k + kAhead < NV) fetch_one(q, k + kAhead);
            if (k >= p.nv) continue;
            bad |= ((x.x + x.y) + (x.z + x.w)) * 0.0f != 0.0f;
            *reinterpret_cast<float4 *>(X + 4 * (lane + kWave * k)) = x;
        }
        return __builtin_amdgcn_ballot_w64(bad) != 0;
    };

    uint32_t i = blockIdx.x;
    if (i >= p.nItems) return;
    Tile cur = tile_of(i);
    fetch(cur, false);
    fetch(cur, true);
    {
        const BufferRsrc none = make_buffer(p.out, 0);
#pragma unroll
        for (int k = 0; k < NV; ++k) buffer_store4(none, (lane + kWave * k) * 16, 0, make_float4(static_cast<float>(k), 0.0f, 0.0f, 0.0f));
    }
    for (;;) {
        const bool chains = stage(cur) || chainsAlways;
        wave_sync();
        const uint32_t iNext = i + gridDim.x;
        const bool more = iNext < p.nItems;
        Tile next = tile_of(more ? iNext : i);
        if (!more) next.nRows = 0;
        fetch(next, false);
        if (chains) {
            for (int e = lane; e < cur.nRows * T; e += kWave) {
                const int r = e / T, t = e - r * T;
                const float *x = p.in + (cur.row0 + r) * T;
                const float *gu = GATED ? p.gate.u + (cur.row0 + r) * T : nullptr;
                const int taps = min(T - t, F);
                float acc = 0.0f;
                for (int k = 0; k < taps; ++k) {
                    acc = __builtin_fmaf(GATED ? x[t + k] * spike_pdf(gu[t + k], p.gate.theta, p.gate.tau, p.gate.gain) : x[t + k],
                                         p.filt[k], acc);
                }
                p.out[(cur.row0 + r) * T + t] = acc * p.Ts;
            }
        } else {
            // step m makes outputs 32 m .. 32 m + 31 from chunks m .. m + NC - 1 and writes them over chunk m
            float *col = X + c * T + 8 * h;
            const float *zeros = X + 16 * T;
            // chunk s of the lane's row; behind the row (where the next row lies), zeros
            auto raw = [&](int s, float4 &v0, float4 &v1) {
                const int t = 32 * s + 8 * h;
                v0 = *reinterpret_cast<const float4 *>(t < T ? col + 32 * s : zeros);
                v1 = *reinterpret_cast<const float4 *>(t + 4 < T ? col + 32 * s + 4 : zeros);
            };
            auto split = [&](const float4 &v0, const float4 &v1) {
                const float x[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
                return split_bf16(x);
            };
            SplitPlanes w[NC];
#pragma unroll
            for (int s = 0; s < NC; ++s) {
                float4 v0, v1;
                raw(s, v0, v1);
                w[s] = split(v0, v1);
            }
            for (int m0 = 0; m0 < nCh; m0 += NC) {
#pragma unroll
                for (int u = 0; u < NC; ++u) {
                    const int m = m0 + u;
                    if (m < nCh) {
                        float4 v0, v1;
                        raw(m + NC, v0, v1);  // the chunk that the next step adds
                        __builtin_amdgcn_sched_barrier(0);
                        // four sums: the leading products and the five smaller ones, of either block
                        f32x4 e0 = {0.0f, 0.0f, 0.0f, 0.0f}, e1 = e0, o0 = e0, o1 = e0;
#pragma unroll
                        for (int s = 0; s < NC; ++s) {
                            const SplitPlanes &x = w[(u + s) % NC];
                            if (s < NCE) e1 = mfma_bf16(aE[s].lo, x.hi, e1);
                            o1 = mfma_bf16(aO[s].lo, x.hi, o1);
                            if (s < NCE) e1 = mfma_bf16(aE[s].hi, x.lo, e1);
                            o1 = mfma_bf16(aO[s].hi, x.lo, o1);
                            if (s < NCE) e1 = mfma_bf16(aE[s].mid, x.mid, e1);
                            o1 = mfma_bf16(aO[s].mid, x.mid, o1);
                            if (s < NCE) e1 = mfma_bf16(aE[s].mid, x.hi, e1);
                            o1 = mfma_bf16(aO[s].mid, x.hi, o1);
                            if (s < NCE) e1 = mfma_bf16(aE[s].hi, x.mid, e1);
                            o1 = mfma_bf16(aO[s].hi, x.mid, o1);
                            if (s < NCE) e0 = mfma_bf16(aE[s].hi, x.hi, e0);
                            o0 = mfma_bf16(aO[s].hi, x.hi, o0);
                        }
                        const int t = 32 * m + 4 * h;
                        if (t < T)
                            *reinterpret_cast<float4 *>(col + 32 * m - 4 * h) =
                                make_float4((e0.x + e1.x) * p.Ts, (e0.y + e1.y) * p.Ts, (e0.z + e1.z) * p.Ts, (e0.w + e1.w) * p.Ts);
                        if (t + 16 < T)
                            *reinterpret_cast<float4 *>(col + 32 * m + 16 - 4 * h) =
                                make_float4((o0.x + o1.x) * p.Ts, (o0.y + o1.y) * p.Ts, (o0.z + o1.z) * p.Ts, (o0.w + o1.w) * p.Ts);
                        w[u] = split(v0, v1);
                    }
                }
            }
        }
        wave_sync();
        fetch(next, true);
        const BufferRsrc bufOut = make_buffer(p.out + cur.row0 * T, chains ? 0 : cur.nRows * T * 4);
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            buffer_store4(bufOut, lane * 16, kWave * 16 * k, *reinterpret_cast<const float4 *>(X + (k < p.nv ? 4 * (lane + kWave * k) : 0)));
            if (k % 8 == 7) __builtin_amdgcn_sched_barrier(0);
        }
        if (!more) break;
        wave_sync();
        i = iNext;
        cur = next;
    }
}

struct MfmaFirPlan {
    int nb, timeTiles, pitch;
};

// Blocks per time tile: whole rows if 16 of them fit into a wavefront's share of LDS, else the fewest tiles.
static MfmaFirPlan plan_mfma(int nBlk, int D, int ldsBytes)
{
    for (int timeTiles = 1; timeTiles <= nBlk; ++timeTiles) {
        const int nb = static_cast<int>(ceil_div(nBlk, timeTiles));
        if (static_cast<int>(ceil_div(nBlk, nb)) != timeTiles) continue;
        const int staged = nb + (timeTiles > 1 ? D - 1 : 0);
        int pitch = 16 * staged;
        if ((pitch / 4) % 2 == 0) pitch += 4;
        if ((16 * pitch + 16) * 4 <= ldsBytes) return MfmaFirPlan{nb, timeTiles, pitch};
        if (nb <= D) break;  // more halo than tile
    }
    return MfmaFirPlan{0, 0, 0};
}

template <int NV>
static void launch_mfma(int D, dim3 grid, size_t lds, hipStream_t st, const MfmaFirArgs &args)
{
#define SLAYER_FIR_MFMA(DD)                                                                                            \
    case DD:                                                                                                           \
        hipLaunchKernelGGL((fir_mfma_kernel<DD, NV>), grid, dim3(64), lds, st, args);                                 \
        break
    switch (D) {
        SLAYER_FIR_MFMA(4);
        SLAYER_FIR_MFMA(5);
        SLAYER_FIR_MFMA(6);
        SLAYER_FIR_MFMA(7);
        SLAYER_FIR_MFMA(8);
        default:
            SLAYER_FIR_MFMA(9);
    }
#undef SLAYER_FIR_MFMA
}

template <bool GATED>
static void launch_split(int nce, int nc, int nv, dim3 grid, size_t lds, hipStream_t st, const MfmaFirArgs &args)
{
#define SLAYER_SPLIT_NV(E, C)                                                                                          \
    if (nv <= 12) hipLaunchKernelGGL((fir_mfma_split_kernel<E, C, 12, GATED>), grid, dim3(64), lds, st, args);        \
    else if (nv <= 16) hipLaunchKernelGGL((fir_mfma_split_kernel<E, C, 16, GATED>), grid, dim3(64), lds, st, args);   \
    else hipLaunchKernelGGL((fir_mfma_split_kernel<E, C, 20, GATED>), grid, dim3(64), lds, st, args)
    if (nc == 3 && nce == 2) { SLAYER_SPLIT_NV(2, 3); }
    else if (nc == 3) { SLAYER_SPLIT_NV(3, 3); }
    else if (nc == 4 && nce == 3) { SLAYER_SPLIT_NV(3, 4); }
    else if (nc == 4) { SLAYER_SPLIT_NV(4, 4); }
    else if (nce == 4) { SLAYER_SPLIT_NV(4, 5); }
    else { SLAYER_SPLIT_NV(5, 5); }
#undef SLAYER_SPLIT_NV
}

bool launch_fir_corr_mfma(float *out, const float *in, const float *filt, int64_t rows, int64_t T, int64_t F, float Ts,
                          const FirGate &gate, hipStream_t stream)
{
    if (F < kFirMfmaMinTaps || F > kFirMfmaMaxTaps || T % 4 != 0 || T < 16 || T > kBufferMaxT) return false;
    if (!aligned16(out) || !aligned16(in) || (gate.u && !aligned16(gate.u))) return false;
    const int D = static_cast<int>((F + 14) / 16 + 1);
    const int nBlk = static_cast<int>(ceil_div(T, 16));
    MfmaFirPlan plan = plan_mfma(nBlk, D, kMfmaLdsBytes);
    if (plan.nb < 1) return false;
    // whole rows whose length spreads the 16 rows over the LDS banks as it is: the tile as it lies in memory
    const bool asInMemory = plan.timeTiles == 1 && (T / 4) % 2 == 1;
    // the gated correlation only in that layout (elsewhere it measured no faster than the tiled kernel)
    if (gate.u && !asInMemory) return false;
    if (asInMemory) plan.pitch = static_cast<int>(T);
    const int64_t items = ceil_div(rows, 16) * plan.timeTiles;
    if (items >= (1LL << 31) || 16 * T >= (1LL << 28)) return false;
    // wavefronts resident at once (8 per compute unit); each walks over its share of the tiles
    const int64_t resident = static_cast<int64_t>(compute_units()) * 8;
    const int64_t trips = ceil_div(items, resident);
    const int64_t waves = ceil_div(ceil_div(items, trips), 8) * 8;  // a multiple of 8: one range of tiles per die
    const int nv = plan.nb + (plan.timeTiles > 1 ? D - 1 : 0);      // vectors per lane = staged blocks per row
    MfmaFirArgs args{out, in, filt, rows, static_cast<int>(T), static_cast<int>(F), plan.nb, plan.timeTiles, plan.pitch,
                     nv, static_cast<uint32_t>(items), Ts, gate};
    const dim3 grid(static_cast<unsigned>(waves));
    // (rows as they lie in memory: every lane writes its nv vectors, nv KiB)
    const size_t lds = asInMemory ? static_cast<size_t>(nv) * 1024 : (static_cast<size_t>(16) * plan.pitch + 16) * sizeof(float);
    if (asInMemory) {
        const int nce = static_cast<int>((15 + F + 31) / 32), nc = static_cast<int>((31 + F + 31) / 32);
        if (gate.u) launch_split<true>(nce, nc, nv, grid, lds, stream, args);
        else launch_split<false>(nce, nc, nv, grid, lds, stream, args);
    } else {
        if (nv <= 12) launch_mfma<12>(D, grid, lds, stream, args);
        else if (nv <= 16) launch_mfma<16>(D, grid, lds, stream, args);
        else launch_mfma<20>(D, grid, lds, stream, args);
    }
    return true;
}

}  // namespace slayer

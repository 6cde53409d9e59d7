// PSP filter and spike function in one kernel, for networks that apply them back to back
// (spike(psp(x)), the ordering of the reference's MLP example):
//
//   u[n][t] = Ts * sum_{i<F} a[n][t-i] * srm[i]        (the causal convolution of fir.hip)
//   then the sequential threshold / refractory loop of spike.hip on u, in place.
//
// Without the round trip of u through memory: 12 bytes per neuron-timestep (read a, write u', write s)
// instead of 20.  Two kernels: filters of 34 to 129 taps on the matrix cores (further down; potentials
// to rounding), all others with the register-window chain - the same values, bit for bit, as
// slayer_conv_f32's chain kernels followed by slayer_get_spikes_f32.  There a 64-lane work-group owns 8 whole rows.  It stages them into LDS reversed in
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


// ---- the same on the matrix cores, for filters of 34 to 129 taps ---------------------------------------------------
// Above about 33 taps the register-window chain is bound by FMA issue.  Here a wavefront owns 16 whole rows and
// filters them as products of a banded Toeplitz matrix of the filter with chunks of 32 samples, on bf16 matrix
// instructions over a three-way split of samples and taps (fir_mfma.hip has the formulation and its error: a few
// 1e-7 of sum |a| |srm|).  The walk goes down in time: the window is the NC chunks up to the one whose 32 outputs
// are made - split once per sample, when the chunk enters - and lane (c = lane % 16, h = lane / 16) supplies samples
// 8h .. 8h + 7 of each chunk of row c and, for block p (16 outputs) of a chunk and the chunk s before it,
// srm[32 s + 16 p + c - (8h + e)].  Its accumulators hold outputs 4h .. 4h + 3 of either block of row c, which it
// writes over the chunk that has just left the window: the membrane potential ends up where the spike walk wants
// it, tile[r][LAG + t].  The candidate bits of the spike walk are set as the outputs are written; the walk (all 64
// lanes, four per row) and the stores are those of spike.hip's row tiles.  The potentials agree with the
// sequential chain to rounding, and the spikes are the spike function of exactly these potentials.  A tile with a
// non-finite sample is filtered as sequential chains instead (a structural zero of the band times an infinity would
// put NaNs where the reference has none), and so is every tile when a tap is not finite.
constexpr int kFusedMfmaRows = 16;
constexpr int kFusedMfmaMaxTaps = 113;  // the first block of a chunk reaches four chunks, the second five

// NC: chunks in the window (the first block of a chunk reaches back 31 + F samples from the chunk's end), NCE: chunks
// that the second block reaches
template <int NCE, int NC, int NU>
__global__ __launch_bounds__(64, 2) void psp_spike_mfma_kernel(float *__restrict__ s, float *__restrict__ u,
                                                            const float *__restrict__ a, const float *__restrict__ srm,
                                                            const float *__restrict__ nu, int64_t rows, int T, int F,
                                                            int nuSize, int P, int MP, float theta, float Ts)
{
    constexpr int R = kFusedMfmaRows, G = 32;
    constexpr int LAG = (NU + 2) & ~3;
    constexpr int NBV = (R * (kFusedMaxT / 4) + kWave - 1) / kWave;  // vectors per lane of a tile, at most
    constexpr int kParts = kWave / R, kRounds = (NU + kParts - 1) / kParts;
    extern __shared__ __align__(16) float lds[];
    float *tile = lds;                                               // [R][P]
    uint32_t *masks = reinterpret_cast<uint32_t *>(lds + R * P);     // [R][MP] spike bits, bit = tile column
    uint32_t *cand = masks + R * MP;                                 // [R][MP] samples at or above the threshold
    float *zeros = reinterpret_cast<float *>(cand + R * MP);         // 64 bytes
    // the refractory kernel with 3 entries in front and room behind, -0.0f (whose addition changes nothing) outside
    float *tapL = zeros + 16 + 3;                                    // [-3, 29)

    const int lane = threadIdx.x;
    const int c = lane & 15, h = lane >> 4;
    const int perRow = T >> 2;
    const float amplitude = 1.0f / Ts;
    const float quiet = __builtin_nanf("");
    const int64_t tiles = (rows + R - 1) / R;

    // A tile is one contiguous run of vectors (rows behind the last one arrive as zeros).  A wavefront walks over
    // tiles; the next tile's samples are on their way into registers while this one is filtered, walked and stored.
    // In three parts.  As many vectors as the registers hold beside the filter's operands and the window (12
    // registers per chunk each) travel during the filter; more of them from then on, during the spike walk, beside
    // the filter's operands and the walk's registers; what is left is fetched while the tile before is stored away
    // and this one is staged, one vector for each one that has been put into LDS.
    constexpr int kWalkRegs = 96 + (NU > 12 ? 16 : 0);   // (measured: the largest counts that leave nothing in scratch)
    constexpr int kRoomWalk = (236 - kWalkRegs - 12 * (NCE + NC)) / 4;
    constexpr int kAhead = kRoomWalk < 1 ? 1 : kRoomWalk < NBV ? kRoomWalk : NBV;
    constexpr int kRoom = (236 - 68 - 12 * (NCE + 2 * NC)) / 4;
    constexpr int kEarly = kRoom < 0 ? 0 : kRoom < kAhead ? kRoom : kAhead;
    float4 x[NBV];
    auto buffer_of = [&](int64_t t) {
        // (behind the tile - or behind the last tile: everything - masked by the range check: a fixed number of
        // memory instructions lets the wait for these loads leave the stores that are issued behind them in flight)
        const int64_t r0 = t < tiles ? t * R : 0;
        const int n = t < tiles ? static_cast<int>(min(static_cast<int64_t>(R), rows - r0)) * perRow : 0;
        return make_buffer(a + r0 * static_cast<int64_t>(T), n * 16);
    };
    auto fetch = [&](int64_t t, bool rest) {
        const BufferRsrc bufA = buffer_of(t);
#pragma unroll
        for (int b = 0; b < kAhead; ++b)
            if ((b >= kEarly) == rest) x[b] = buffer_load4(bufA, (lane + b * kWave) * 16, 0);
    };
    // the lane index behind a barrier for the optimiser: the (row, vector) sequences of the staging and storing
    // loops do not depend on the tile, and kept across the filter and the walk they would cost 2 registers per vector
    auto lane_again = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    int64_t tileIdx = blockIdx.x;
    if (tileIdx >= tiles) return;
    fetch(tileIdx, false);
    fetch(tileIdx, true);
    // the lane's part of the Toeplitz factor, split; the range check of a buffer that ends with the filter turns every
    // index that is not a tap into a zero.  aE: the operand of a chunk's second block, which reaches NCE chunks; aO:
    // of its first block, which reaches all NC.
    SplitPlanes aE[NCE], aO[NC];
    bool chainsAlways = false;
    {
        const BufferRsrc bufF = make_buffer(srm, F * 4);
        bool badTap = false;
#pragma unroll
        for (int sc = 0; sc < NC; ++sc) {
            float fe[8], fo[8];
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int tapE = 32 * sc + 16 + c - (8 * h + e), tapO = tapE - 16;
                fe[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bufF, masked_offset(tapE >= 0 && tapE < F, tapE * 4), 0, 0));
                fo[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(bufF, masked_offset(tapO >= 0 && tapO < F, tapO * 4), 0, 0));
                badTap |= fe[e] * 0.0f != 0.0f || fo[e] * 0.0f != 0.0f;
            }
            if (sc < NCE) aE[sc] = split_bf16(fe);
            aO[sc] = split_bf16(fo);
        }
        chainsAlways = __builtin_amdgcn_ballot_w64(badTap) != 0;
    }
    float tap[NU];
#pragma unroll
    for (int j = 0; j < NU; ++j) tap[j] = (j < nuSize) ? nu[j] : -0.0f;
    float myTap[kRounds];  // this lane's taps in the candidate walk (lane p of a row: taps p kRounds ... )
#pragma unroll
    for (int j = 0; j < kRounds; ++j) {
        const int tj = (lane % kParts) * kRounds + j;
        myTap[j] = tj < nuSize ? nu[tj] : -0.0f;
    }
    // a refractory kernel without positive taps only lowers the potential: samples below the threshold never fire
    bool monotone = true;
#pragma unroll
    for (int j = 0; j < NU; ++j) monotone = monotone && tap[j] <= 0.0f;

    if (lane < 4) *reinterpret_cast<float4 *>(zeros + 4 * lane) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (lane < 32) tapL[lane - 3] = (lane >= 3 && lane - 3 < nuSize) ? nu[lane - 3] : -0.0f;
    for (;;) {
    const int64_t row0 = tileIdx * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), rows - row0));
    const int nVec = nRows * perRow;
    for (int i = lane; i < R * MP; i += kWave) cand[i] = 0u;
    bool bad = false;
    {
        const BufferRsrc bufCur = buffer_of(tileIdx);
        RowCol rc;
        rc.init(lane_again(), perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NBV; ++b) {
            if (lane + b * kWave < R * perRow) {
                *reinterpret_cast<float4 *>(tile + rc.r * P + LAG + (rc.c << 2)) = x[b];
                // infinite or NaN (or four samples that add up to more than fp32 holds, which only costs time)
                bad |= ((x[b].x + x[b].y) + (x[b].z + x[b].w)) * 0.0f != 0.0f;
            }
            if (b + kAhead < NBV) x[b + kAhead] = buffer_load4(bufCur, (lane + (b + kAhead) * kWave) * 16, 0);
            rc.advance(dr, dc, perRow);
        }
    }
    const bool chains = __builtin_amdgcn_ballot_w64(bad) != 0 || chainsAlways;
    wave_sync();
    const int64_t tileNext = tileIdx + gridDim.x;
    fetch(tileNext, false);

    auto mark4 = [&](int r, int col, const float4 &y) {  // col is a multiple of 4: the four bits lie in one word
        const uint32_t bits = (y.x >= theta ? 1u : 0u) | (y.y >= theta ? 2u : 0u) | (y.z >= theta ? 4u : 0u) |
                              (y.w >= theta ? 8u : 0u);
        if (bits) atomicOr(cand + r * MP + (col >> 5), bits << (col & 31));
    };
    if (chains) {
        // a non-finite sample: the tile's potentials as sequential chains over the valid taps, from memory
        for (int e = lane; e < nVec; e += kWave) {
            const int r = e / perRow, t0 = (e - r * perRow) << 2;
            const float *xr = a + (row0 + r) * static_cast<int64_t>(T);
            float y[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int t = t0 + k;
                const int taps = min(t + 1, F);
                float acc = 0.0f;
                for (int i = 0; i < taps; ++i) acc = __builtin_fmaf(xr[t - i], srm[i], acc);
                y[k] = acc * Ts;
            }
            const float4 q = make_float4(y[0], y[1], y[2], y[3]);
            *reinterpret_cast<float4 *>(tile + r * P + LAG + t0) = q;
            if (monotone) mark4(r, LAG + t0, q);
        }
    } else {
        // walk down in time: a step makes outputs 32 m .. 32 m + 31 from chunks m - NC + 1 .. m and writes them over
        // chunk m
        const int nCh = (T + 31) >> 5;
        float *col = tile + c * P + LAG + 8 * h;
        // chunk q of the lane's row; zeros before the row's start and behind its end
        auto raw = [&](int q, float4 &v0, float4 &v1) {
            const int t = 32 * q + 8 * h;
            v0 = *reinterpret_cast<const float4 *>(q >= 0 && t < T ? col + 32 * q : zeros);
            v1 = *reinterpret_cast<const float4 *>(q >= 0 && t + 4 < T ? col + 32 * q + 4 : zeros);
        };
        auto split = [&](const float4 &v0, const float4 &v1) {
            const float xs[8] = {v0.x, v0.y, v0.z, v0.w, v1.x, v1.y, v1.z, v1.w};
            return split_bf16(xs);
        };
        SplitPlanes w[NC];  // at step k of a round, w[(k + sc) % NC] holds chunk m - sc
#pragma unroll
        for (int sc = 0; sc < NC; ++sc) {
            float4 v0, v1;
            raw(nCh - 1 - sc, v0, v1);
            w[sc] = split(v0, v1);
        }
        for (int j0 = 0; j0 < nCh; j0 += NC) {
#pragma unroll
            for (int k = 0; k < NC; ++k) {
                if (j0 + k < nCh) {
                    const int m = nCh - 1 - (j0 + k);
                    float4 v0, v1;
                    raw(m - NC, v0, v1);                // the chunk that the next step adds
                    __builtin_amdgcn_sched_barrier(0);  // (issued here, not after the step's matrix work)
                    // four sums: the leading products and the five smaller ones, of either block
                    f32x4 e0 = {0.0f, 0.0f, 0.0f, 0.0f}, e1 = e0, o0 = e0, o1 = e0;
#pragma unroll
                    for (int sc = 0; sc < NC; ++sc) {
                        const SplitPlanes &xs = w[(k + sc) % NC];
                        if (sc < NCE) e1 = mfma_bf16(aE[sc].lo, xs.hi, e1);
                        o1 = mfma_bf16(aO[sc].lo, xs.hi, o1);
                        if (sc < NCE) e1 = mfma_bf16(aE[sc].hi, xs.lo, e1);
                        o1 = mfma_bf16(aO[sc].hi, xs.lo, o1);
                        if (sc < NCE) e1 = mfma_bf16(aE[sc].mid, xs.mid, e1);
                        o1 = mfma_bf16(aO[sc].mid, xs.mid, o1);
                        if (sc < NCE) e1 = mfma_bf16(aE[sc].mid, xs.hi, e1);
                        o1 = mfma_bf16(aO[sc].mid, xs.hi, o1);
                        if (sc < NCE) e1 = mfma_bf16(aE[sc].hi, xs.mid, e1);
                        o1 = mfma_bf16(aO[sc].hi, xs.mid, o1);
                        if (sc < NCE) e0 = mfma_bf16(aE[sc].hi, xs.hi, e0);
                        o0 = mfma_bf16(aO[sc].hi, xs.hi, o0);
                    }
                    const int t = 32 * m + 4 * h;   // the lane's outputs: t .. t + 3 (first block), t + 16 .. (second)
                    if (t < T) {
                        const float4 y = make_float4((o0.x + o1.x) * Ts, (o0.y + o1.y) * Ts, (o0.z + o1.z) * Ts, (o0.w + o1.w) * Ts);
                        *reinterpret_cast<float4 *>(col + 32 * m - 4 * h) = y;
                        if (monotone) mark4(c, LAG + t, y);
                    }
                    if (t + 16 < T) {
                        const float4 y = make_float4((e0.x + e1.x) * Ts, (e0.y + e1.y) * Ts, (e0.z + e1.z) * Ts, (e0.w + e1.w) * Ts);
                        *reinterpret_cast<float4 *>(col + 32 * m + 16 - 4 * h) = y;
                        if (monotone) mark4(c, LAG + t + 16, y);
                    }
                    w[k] = split(v0, v1);
                }
            }
        }
    }
    fetch(tileNext, true);
    wave_sync();

    // ---- walk: columns [0, T + LAG) of the tile become final
    const int Wc = T + LAG;
    const int words = (Wc + 31) >> 5;
    const int cr = lane / kParts, part = lane - cr * kParts;
    bool hop = monotone;
    uint32_t nzw = 0u;  // bit w: word w of the row has candidates
    if (monotone) {
        int mine = 0;
        for (int wd = part; wd < words; wd += kParts) {
            const uint32_t cw = cand[cr * MP + wd];
            mine += __builtin_popcount(cw);
            nzw |= (cw != 0u ? 1u : 0u) << wd;
        }
#pragma unroll
        for (int off = kParts / 2; off > 0; off >>= 1) {
            mine += __shfl_xor(mine, off, kWave);
            nzw |= __shfl_xor(nzw, off, kWave);
        }
        // from candidate to candidate while no row of the tile has more than one per 12 samples (the wavefront
        // stays as long as its busiest row)
        hop = __builtin_amdgcn_ballot_w64(mine * 12 > Wc) == 0;
    }
    if (hop) {
        // every lane of a row follows the row's candidates; on a spike each adds its own taps of the response
        const uint32_t *cw = cand + cr * MP;
        uint32_t *mw = masks + cr * MP;
        float *mine = tile + cr * P;
        for (int wd = part; wd < words; wd += kParts) mw[wd] = 0u;  // words without candidates have no spikes
        int wd = 0;
        uint32_t cm = 0u, fired = 0u;
        while (__builtin_amdgcn_ballot_w64((cm | nzw) != 0u) != 0) {
            if (cm == 0u && nzw != 0u) {  // on to the row's next word with candidates
                if (fired != 0u) mw[wd] = fired;
                fired = 0u;
                wd = __builtin_ctz(nzw);
                nzw &= nzw - 1u;
                cm = cw[wd];
            }
            if (cm != 0u) {
                const int k = __builtin_ctz(cm);
                cm &= cm - 1u;
                // the candidate itself (the same address for the row's lanes) and this lane's samples of the response
                // in one round of reads: a walk is as long as the chain of its LDS round trips
                const float *q0 = mine + (wd << 5) + k;
                float *q = mine + (wd << 5) + k + part * kRounds;
                const float x0 = *q0;
                float val[kRounds];
#pragma unroll
                for (int j = 0; j < kRounds; ++j)
                    if (part * kRounds + j < NU) val[j] = q[j];   // (what lies behind the response belongs to the next row)
                if (x0 >= theta) {
                    fired |= 1u << k;
#pragma unroll
                    for (int j = 0; j < kRounds; ++j)
                        if (part * kRounds + j < NU) q[j] = val[j] + myTap[j];
                }
            }
        }
        if (fired != 0u) mw[wd] = fired;
    } else {
        // Every sample in turn, 32 samples at a time through a register window of 32 + LAG samples, as in spike.hip -
        // but the window of a row is spread over the row's four lanes, lane p keeping the samples whose window index
        // is p (mod 4).  The sample under test is broadcast within the quad (a lane-permuting move, no LDS); on a
        // spike every lane adds the taps that fall on its own samples, NA instead of NU additions.
        constexpr int NW = (G + LAG) / kParts;          // window registers per lane
        constexpr int NA = (NU + kParts - 1) / kParts + 1;  // additions per spike and lane
        float wq[NW];    // wq[m] = window sample 4 m + part
        float tq[kParts][NA];  // tq[res][i] = nu[4 i + part - res]: what a spike at window index k = res (mod 4) adds to wq[k / 4 + i]
#pragma unroll
        for (int res = 0; res < kParts; ++res)
#pragma unroll
            for (int i = 0; i < NA; ++i) tq[res][i] = tapL[4 * i + part - res];
        float *mine = tile + cr * P;
#pragma unroll
        for (int m = 0; m < LAG / kParts; ++m) wq[m] = quiet;
        const int groups = (Wc + G - 1) / G;
        for (int g = 0; g < groups; ++g) {
            const int c0 = g * G;
            if (c0 + G <= T) {
#pragma unroll
                for (int m = 0; m < G / kParts; ++m) wq[LAG / kParts + m] = mine[LAG + c0 + 4 * m + part];
            } else {
#pragma unroll
                for (int m = 0; m < G / kParts; ++m)
                    wq[LAG / kParts + m] = (c0 + 4 * m + part < T) ? mine[LAG + c0 + 4 * m + part] : quiet;
            }
            uint32_t fired = 0;
            auto sample = [&](int k) {  // window sample k, from the lane of the quad that keeps it
                constexpr int kQuad[4] = {0x00, 0x55, 0xaa, 0xff};  // quad_perm: all four lanes read lane k % 4
                const int bitsIn = __builtin_bit_cast(int, wq[k / kParts]);
                int bitsOut = 0;
                switch (k % kParts) {
                    case 0: bitsOut = __builtin_amdgcn_update_dpp(0, bitsIn, kQuad[0], 0xf, 0xf, false); break;
                    case 1: bitsOut = __builtin_amdgcn_update_dpp(0, bitsIn, kQuad[1], 0xf, 0xf, false); break;
                    case 2: bitsOut = __builtin_amdgcn_update_dpp(0, bitsIn, kQuad[2], 0xf, 0xf, false); break;
                    default: bitsOut = __builtin_amdgcn_update_dpp(0, bitsIn, kQuad[3], 0xf, 0xf, false); break;
                }
                return __builtin_bit_cast(float, bitsOut);
            };
#pragma unroll
            for (int k = 0; k < G; k += 2) {
                // one scalar branch per two samples (the second sample is tested again inside, after the first one's
                // refractory response)
                const float xa = sample(k), xb = sample(k + 1);
                if (__builtin_amdgcn_ballot_w64((xa >= theta) | (xb >= theta)) != 0) {
                    if (xa >= theta) {
                        fired |= 1u << k;
#pragma unroll
                        for (int i = 0; i < NA; ++i) wq[k / kParts + i] += tq[k % kParts][i];
                    }
                    if (sample(k + 1) >= theta) {
                        fired |= 2u << k;
#pragma unroll
                        for (int i = 0; i < NA; ++i) wq[(k + 1) / kParts + i] += tq[(k + 1) % kParts][i];
                    }
                }
            }
#pragma unroll
            for (int m = 0; m < G / kParts; ++m) mine[c0 + 4 * m + part] = wq[m];
            masks[cr * MP + g] = fired;  // (the same word from the four lanes of a row)
#pragma unroll
            for (int m = 0; m < LAG / kParts; ++m) wq[m] = wq[G / kParts + m];
        }
    }
    wave_sync();

    // ---- retire: u' and s of the whole tile, one contiguous run (a fixed number of stores, masked by the buffers'
    //      range check: the wait for the next tile's loads, which are older, can then leave exactly these in flight)
    {
        const BufferRsrc bufU = make_buffer(u + row0 * static_cast<int64_t>(T), nVec * 16);
        const BufferRsrc bufS = make_buffer(s + row0 * static_cast<int64_t>(T), nVec * 16);
        RowCol rc;
        rc.init(lane_again(), perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NBV; ++b) {
            const int r = min(rc.r, R - 1);  // (lanes behind the tile: their stores are dropped)
            const int cl = LAG + (rc.c << 2);
            const uint32_t m = masks[r * MP + (cl >> 5)] >> (cl & 31);
            buffer_store4(bufU, (lane + b * kWave) * 16, 0, *reinterpret_cast<const float4 *>(tile + r * P + cl));
            buffer_store4(bufS, (lane + b * kWave) * 16, 0,
                          make_float4((m & 1u) ? amplitude : 0.0f, (m & 2u) ? amplitude : 0.0f,
                                      (m & 4u) ? amplitude : 0.0f, (m & 8u) ? amplitude : 0.0f));
            rc.advance(dr, dc, perRow);
            if (b % 4 == 3) __builtin_amdgcn_sched_barrier(0);  // a few vectors at a time: they occupy registers
        }
    }
    if (tileNext >= tiles) break;
    wave_sync();
    tileIdx = tileNext;
    }
}

template <int NU>
static int launch_psp_spike_mfma(float *s, float *u, const float *a, const float *srm, const float *nu, int64_t rows,
                                 int T, int F, int nuSize, float theta, float Ts, hipStream_t st)
{
    constexpr int LAG = (NU + 2) & ~3;
    // a row of the tile: LAG columns in front, the samples, and room for the response of a spike in the last sample
    // (hop walk) or for whole groups of 32 (window walk); a pitch of 4 (mod 32) spreads the 16 rows over the banks
    int P = LAG + T + NU;
    if (P < ((T + LAG + 31) & ~31)) P = (T + LAG + 31) & ~31;
    P = ((P - 4 + 31) & ~31) + 4;
    const int MP = (T + LAG + 31) / 32 + 1;
    const size_t lds = (static_cast<size_t>(kFusedMfmaRows) * P + 2 * kFusedMfmaRows * MP + 16 + 32) * sizeof(float);
    // wavefronts resident at once (what the tiles' LDS leaves room for); each walks over its share of the tiles
    const int64_t tiles = ceil_div(rows, kFusedMfmaRows);
    const int64_t perUnit = 160 * 1024 / static_cast<int64_t>(lds);
    const int64_t resident = static_cast<int64_t>(compute_units()) * (perUnit < 8 ? perUnit : 8);
    const int64_t trips = ceil_div(tiles, resident);
    const dim3 grid(static_cast<unsigned>(ceil_div(tiles, trips)));
    const int nce = (15 + F + 31) / 32, nc = (31 + F + 31) / 32;
#define SLAYER_PSP_SPIKE_MFMA(E, C)                                                                                   \
    hipLaunchKernelGGL((psp_spike_mfma_kernel<E, C, NU>), grid, dim3(kWave), lds, st, s, u, a, srm, nu, rows, T, F,   \
                       nuSize, P, MP, theta, Ts)
    if (nc == 3 && nce == 2) SLAYER_PSP_SPIKE_MFMA(2, 3);
    else if (nc == 3) SLAYER_PSP_SPIKE_MFMA(3, 3);
    else if (nc == 4 && nce == 3) SLAYER_PSP_SPIKE_MFMA(3, 4);
    else if (nc == 4) SLAYER_PSP_SPIKE_MFMA(4, 4);
    else SLAYER_PSP_SPIKE_MFMA(4, 5);
#undef SLAYER_PSP_SPIKE_MFMA
    return launch_status();
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
    // (from 114 taps on the filter's operands, five chunks for either block, leave the fused kernel no registers for a
    // tile in flight: the two kernels then)
    if (F > kFusedMfmaMaxTaps && F <= kFirMfmaMaxTaps && T >= 16) {
        const int status = slayer_conv_f32(u, a, srm, nNeurons, T, F, Ts, stream);
        if (status != SLAYER_OK) return status;
        return slayer_get_spikes_f32(s, u, nu, nNeurons, T, nuSize, theta, Ts, stream);
    }
    if (F >= kFirMfmaMinTaps && F <= kFusedMfmaMaxTaps && T >= 16) {  // filters that pay on the matrix cores
        if (nuSize <= 12)
            return launch_psp_spike_mfma<12>(s, u, a, srm, nu, nNeurons, static_cast<int>(T), static_cast<int>(F),
                                             static_cast<int>(nuSize), theta, Ts, st);
        return launch_psp_spike_mfma<24>(s, u, a, srm, nu, nNeurons, static_cast<int>(T), static_cast<int>(F),
                                         static_cast<int>(nuSize), theta, Ts, st);
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

// Temporal FIR of neuron rows on the matrix cores, for dense input and filters of 34 to 129 taps, where the
// register-window kernels of fir.hip are bound by FMA issue (an FIR of 77 taps needs 154 flop per 8 bytes).
// Correlation only (plain, or with the spike function's surrogate gradient applied to the samples on their way
// into LDS): the convolution's input is mostly spike trains, which the tiled kernel of fir.hip serves through
// its event-driven path.
//
// The rows are cut into blocks of 16 samples.  For Y[m] = sum_t X[m+t] * filt[t], the 16 outputs of block b of
// 16 rows are the 16x16 product
//
//     Y[16b + i][row c] = sum_{d < D} sum_{kk < 16}  filt[16d + kk - i] * X[16(b + d) + kk][row c]
//
// of a banded Toeplitz matrix made of the filter (zero where 16d + kk - i is not a tap) and the D = F/16 + 1..2
// input blocks from b on.  v_mfma_f32_16x16x4_f32 takes 4 of the 16 kk per instruction: a lane (c = lane % 16,
// h = lane / 16) supplies X[.. + 4h + v] of row c for instruction v = 0..3, which are the four components of ONE
// 16-byte LDS read, and filt[16d + 4h + v - i] for i = lane % 16, which it keeps in 4 D registers.  Its accumulator
// then holds outputs 4h..4h+3 of row c.
//
// A work-group is ONE wavefront that walks over tiles of 16 consecutive rows (all of their samples, or a tile of
// their time axis plus D - 1 blocks of halo).  It copies a tile into LDS with 16-byte loads that run through the
// rows' memory front to back, walks the blocks - from one block to the next the window moves by one block, so each
// step reads one new block from LDS and the window registers rotate (the walk is unrolled by the window size) -
// writes every output block over the input block that has just left the window, and copies the rows back out the
// way they came in.  The next tile's samples are on their way into registers during the walk.  No barriers: the
// wavefronts of a compute unit overlap each other's memory and matrix work.
//
// The matrix instruction sums 4 products per step in its own order, so results agree with the sequential
// chain to rounding (about 1e-7 relative), not bit for bit.  A structural zero times a non-finite sample
// would be NaN where the chain has no such term: a wavefront that meets a non-finite sample computes its
// outputs with the sequential chain over the valid taps instead.
#include "common.h"
#include "fir_core.h"

namespace slayer {

typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMfmaLdsBytes = 160 * 1024 / 8;  // per wavefront: 8 of them on a compute unit

struct MfmaFirArgs {
    float *out;
    const float *in, *filt;
    int64_t rows;
    int T, F;
    int nb;         // output blocks per tile of the time axis
    int timeTiles;  // tiles per row
    int pitch;      // floats per row in LDS; pitch / 4 is odd, which spreads the 16 rows over the banks
    int nv;         // 16-byte vectors per lane and tile that are in use (<= NV)
    uint32_t nItems;
    float Ts;
    FirGate gate;  // GATED: the samples are in * gain * exp(-|u - theta| / tau), applied on the way into LDS
};

// NV: 16-byte vectors per lane and tile, NV * 64 >= 16 rows * (staged blocks * 4)
// LINEAR: the tile is 16 whole rows kept in LDS exactly as they lie in memory (pitch == T): vector e of the tile
// is vector e of LDS, no index arithmetic, and the range check of the buffers masks what lies behind the last row.
// The last block of a row then ends in the first samples of the next row, which the walk masks.
template <int D, int NV, bool LINEAR, bool GATED>
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
    float4 pre[NV], preU[GATED ? NV : 1];
    constexpr int kEarlyU = (GATED && LINEAR) ? NV / 2 : NV;   // potentials fetched ahead with the samples (LINEAR is the only gated layout)
    // the lane index behind a barrier for the optimiser: the (row, vector) sequences below do not depend on the
    // tile, and kept across the walk they would cost 2 registers per vector
    auto lane_again = [&]() {
        int l = lane;
        asm volatile("" : "+v"(l));
        return l;
    };
    auto fetch = [&](const Tile &q) {
        if (LINEAR) {
            const BufferRsrc bufIn = make_buffer(p.in + q.row0 * T, q.nRows * T * 4);
            const BufferRsrc bufU = make_buffer(GATED ? p.gate.u + q.row0 * T : p.in, q.nRows * T * 4);
            // (all NV of them, whatever p.nv is: the vectors behind the 16 rows fail the buffers' range check and cost
            // nothing, and a fixed number of loads and stores per tile is what lets the wait for a tile's loads leave
            // the younger stores of the tile before it in flight)
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                // (the vector's number travels in the instruction's scalar offset: one address register for all of them)
                pre[k] = buffer_load4(bufIn, lane * 16, kWave * 16 * k);
                // (the potentials of the tile's second half are fetched by stage(), while it gates the first half: with
                // both tensors of a whole tile in registers during the walk, the 110-tap kernel spilled)
                if (GATED && k < kEarlyU) preU[k] = buffer_load4(bufU, lane * 16, kWave * 16 * k);
            }
            return;
        }
        const BufferRsrc bufIn = make_buffer(p.in + q.row0 * T);
        const BufferRsrc bufU = make_buffer(GATED ? p.gate.u + q.row0 * T : p.in);
        RowCol rc;
        rc.init(lane_again(), lenIn, 1.0f / static_cast<float>(lenIn));
        const int dr = kWave / lenIn, dc = kWave % lenIn;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            const int t = q.t0 + (rc.c << 2);
            const int off = masked_offset(rc.r < q.nRows && t < T, (rc.r * T + t) * 4);
            pre[k] = buffer_load4(bufIn, off, 0);
            if (GATED) preU[k] = buffer_load4(bufU, off, 0);
            rc.advance(dr, dc, lenIn);
        }
    };
    auto stage = [&](const Tile &q) {  // the fetched vectors into LDS; true if a sample is not finite
        bool bad = false;
        if (GATED && LINEAR) {
            const BufferRsrc bufU = make_buffer(p.gate.u + q.row0 * T, q.nRows * T * 4);
#pragma unroll
            for (int k = kEarlyU; k < NV; ++k) preU[k] = buffer_load4(bufU, lane * 16, kWave * 16 * k);
        }
        RowCol rc;
        if (!LINEAR) rc.init(lane_again(), lenIn, 1.0f / static_cast<float>(lenIn));
        const int dr = kWave / lenIn, dc = kWave % lenIn;
#pragma unroll
        for (int k = 0; k < NV; ++k) {
            if (LINEAR && k >= p.nv) continue;
            float4 x = pre[k];
            if (GATED)
                x = make_float4(x.x * spike_pdf(preU[k].x, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.y * spike_pdf(preU[k].y, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.z * spike_pdf(preU[k].z, p.gate.theta, p.gate.tau, p.gate.gain),
                                x.w * spike_pdf(preU[k].w, p.gate.theta, p.gate.tau, p.gate.gain));
            // infinite or NaN (or four samples that add up to more than fp32 holds, which only costs time)
            bad |= ((x.x + x.y) + (x.z + x.w)) * 0.0f != 0.0f;
            if (LINEAR) {
                *reinterpret_cast<float4 *>(X + 4 * (lane + kWave * k)) = x;
            } else {
                if (rc.r < 16) *reinterpret_cast<float4 *>(X + rc.r * P + (rc.c << 2)) = x;
                rc.advance(dr, dc, lenIn);
            }
        }
        return __builtin_amdgcn_ballot_w64(bad) != 0;
    };

    // 64 bytes of zeros: behind the 16 rows, where the linear copy leaves zeros with every tile (the range check of
    // its loads; nv KiB hold at least 256 bytes more than 16 rows whose T / 4 is odd), else an extra block
    const int zeroOff = LINEAR ? 16 * T : 16 * P;
    if (!LINEAR && lane < 4) *reinterpret_cast<float4 *>(X + zeroOff + 4 * lane) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

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
        const bool chains = stage(cur);
        wave_sync();
        const uint32_t iNext = i + gridDim.x;
        const bool more = iNext < p.nItems;
        // (the next tile's loads behind every wait of stage(): moved up between them, as the compiler likes to do to
        // reuse the registers one by one, each of those waits would also wait for the stores of the tile before)
        // (behind the last tile: a tile without rows, whose loads all fail the range check)
        Tile next = tile_of(more ? iNext : i);
        if (!more) next.nRows = 0;
        fetch(next);
        if (chains) {
            // a non-finite sample: the tile's outputs as sequential chains over the valid taps
            const int width = min(16 * cur.nb, T - cur.t0);
            for (int e = lane; e < cur.nRows * width; e += kWave) {
                const int r = e / width, t = cur.t0 + (e - r * width);
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
            // walk: step j makes output block j from input blocks j .. j + D - 1 and writes it over input block j
            float *col = X + c * P + 4 * h;
            const float *zeros = X + zeroOff + 4 * h;
            const int nIn = cur.nIn;
            // block q of the lane's row; behind the row, 16 bytes of zeros (choosing the address instead of masking
            // the data leaves nothing to do when the read returns, so it can stay in flight during the step)
            auto block = [&](int q) {
                const bool keep = q < nIn && (!LINEAR || 16 * q + 4 * h < T);
                return *reinterpret_cast<const float4 *>(keep ? col + 16 * q : zeros);
            };
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
                        if (!LINEAR || 16 * j + 4 * h < T)  // (behind the row lies the next row)
                            *reinterpret_cast<float4 *>(col + 16 * j) =
                                make_float4(acc.x * p.Ts, acc.y * p.Ts, acc.z * p.Ts, acc.w * p.Ts);
                    }
                }
            }
        }
        wave_sync();
        // rows back out (a fixed number of stores, masked: the wait for the next tile's loads, which are older,
        // can then leave exactly these in flight)
        if (LINEAR) {
            const BufferRsrc bufOut = make_buffer(p.out + cur.row0 * T, chains ? 0 : cur.nRows * T * 4);
#pragma unroll
            for (int k = 0; k < NV; ++k) {
                // (vectors from p.nv on lie behind the 16 rows: read from the tile's first bytes, dropped by the range check)
                buffer_store4(bufOut, lane * 16, kWave * 16 * k, *reinterpret_cast<const float4 *>(X + (k < p.nv ? 4 * (lane + kWave * k) : 0)));
                if (k % 8 == 7) __builtin_amdgcn_sched_barrier(0);  // a few vectors at a time: they occupy registers
            }
        } else {
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

template <int NV, bool LINEAR, bool GATED>
static void launch_mfma(int D, dim3 grid, size_t lds, hipStream_t st, const MfmaFirArgs &args)
{
#define SLAYER_FIR_MFMA(DD)                                                                                            \
    case DD:                                                                                                           \
        hipLaunchKernelGGL((fir_mfma_kernel<DD, NV, LINEAR, GATED>), grid, dim3(64), lds, st, args);                  \
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
    const bool linear = plan.timeTiles == 1 && (T / 4) % 2 == 1;
    // the gated correlation only in that layout (elsewhere it measured no faster than the tiled kernel)
    if (gate.u && !linear) return false;
    if (linear) plan.pitch = static_cast<int>(T);
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
    // (the linear layout writes whole vectors per lane: nv KiB)
    const size_t lds = linear ? static_cast<size_t>(nv) * 1024 : (static_cast<size_t>(16) * plan.pitch + 16) * sizeof(float);
    if (gate.u) {
        if (nv <= 12) launch_mfma<12, true, true>(D, grid, lds, stream, args);
        else if (nv <= 16) launch_mfma<16, true, true>(D, grid, lds, stream, args);
        else launch_mfma<20, true, true>(D, grid, lds, stream, args);
    } else if (linear) {
        if (nv <= 12) launch_mfma<12, true, false>(D, grid, lds, stream, args);
        else if (nv <= 16) launch_mfma<16, true, false>(D, grid, lds, stream, args);
        else launch_mfma<20, true, false>(D, grid, lds, stream, args);
    } else {
        if (nv <= 12) launch_mfma<12, false, false>(D, grid, lds, stream, args);
        else if (nv <= 16) launch_mfma<16, false, false>(D, grid, lds, stream, args);
        else launch_mfma<20, false, false>(D, grid, lds, stream, args);
    }
    return true;
}

}  // namespace slayer

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
// Short refractory kernels (nuSize <= 24, the normal case) take the row-tile kernel further
// down instead: fewer rows per wavefront, long contiguous runs per row, and a per-lane register
// window in place of the ring.
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
        wave_sync();

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
        wave_sync();

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
        wave_sync();
    }
}

// ---- row-tile kernel (nuSize <= NU) --------------------------------------------------------------------
// The fast path.  A wavefront owns R consecutive rows and moves them through LDS in
// pieces of Tc samples per row (the whole row when it is short enough), so that global memory
// is read and written as long contiguous runs with 16-byte accesses per lane - the access
// pattern of a plain copy.  The sequential part then works in LDS, lane = row:
//  * a refractory kernel without positive taps (the normal case) can only lower the potential, so a sample
//    that arrives below the threshold never fires.  All 64 lanes mark the samples at or above it
//    ("candidates", a few per cent) while the piece is staged, one bit per sample, and the walking lanes go from
//    candidate to candidate: test the sample's current value and, on a spike, add nu[0..NU) onto the NU samples
//    from it on, in place - the same fp32 additions in the same order as the sequential loop - and strike the
//    samples that the response has taken below the threshold from the candidates;
//  * any other kernel, and tiles with a row that is above the threshold half of the time or more: every
//    sample in turn through a register window that is spread over the lanes of the row (further down).
// The last LAG samples of a piece are not final until the next piece arrives: they (and their candidate bits)
// are copied to the front of the tile and open the next piece.  Taps beyond nuSize are -0.0f, whose addition
// changes no value; a response may reach past the row's end into padding that is never stored.
// Short tiles keep many wavefronts (and bytes) in flight per CU; the walking wavefront shares its SIMD's issue
// slots with those that move data, so both walks use all 64 lanes (64 / R per row) to need fewer instructions.
constexpr int kTileMaxPiece = 352;  // longest row (samples) that travels whole
// Rows in pieces: samples per piece and row.  With 8-row tiles - tensors of few, long rows - the bytes in flight
// per compute unit are what the rows in LDS amount to, so those pieces are longer.
constexpr int kTilePiece16 = 256, kTilePiece8 = 512;
constexpr int kSpikeRecordMaxT = 16384;  // longest row in pieces whose spikes can be stored shifted (2 KiB of spike bits)

// LAG: samples of a piece that stay behind for the next one (>= NU - 1, whole 16-byte vectors; 32 = one word of
// candidate bits for rows in pieces).  The samples that leave a piece are the ones LAG before its end, so with
// several pieces per row LAG = 32 keeps every run of stores on 128-byte boundaries of the row (partial lines
// are expensive to write).
// R: rows per tile (16, or 8 when the tensor has too few rows to fill the GPU with 16-row tiles).
// MODE: how global memory is accessed.  kTileVec: rows are whole 16-byte vectors.  kTileFlat:
// they are not (T % 4 != 0), but the rows of a tile travel whole and an 8-row tile is one
// contiguous, 16-byte aligned run of whole vectors, so it is still moved with 16-byte accesses;
// a vector may then hold the end of one row and the start of the next, and its four samples are
// placed into (gathered from) LDS one by one.  kTileScalar: anything else, one sample per access.
constexpr int kTileScalar = 0, kTileVec = 1, kTileFlat = 2;

// Optional time shift of the spike output (the delayShift that follows spike() in networks with
// axonal delays, fused into the store of the spikes): s[t] = spike[t - k], k = (int)(delay / Ts),
// with one delay for all rows or one per neuron of a batch item (row % lutSize).  The membrane
// potential is not shifted.  Tiles whose rows travel whole read the shifted bits from the tile's masks; rows in
// pieces keep the spike bits of the whole row in LDS (rows of whole vectors up to kSpikeRecordMaxT samples).
struct SpikeDelay {
    const float *lut;   // per-neuron delays, or NULL
    int64_t lutSize;    // neurons per batch item when lut is given
    float delay;        // the one delay when lut is NULL
    float Ts;
    int on;
};

template <int NU, int MODE, int LAG, int R>
__global__ __launch_bounds__(64) void spike_tile_kernel(float *__restrict__ s, float *u,
                                                        const float *__restrict__ nu, int64_t rows,
                                                        int T, int nuSize, int Tc, int P, int MP, int MPT,
                                                        int64_t tiles, float theta, float Ts, SpikeDelay dl)
{
    static_assert(LAG >= NU - 1 && LAG % 4 == 0, "the window must cover the refractory kernel");
    constexpr bool VEC = MODE == kTileVec, FLAT = MODE == kTileFlat;
    constexpr int V = VEC ? 4 : 1;      // samples per (row-wise) global access
    // longest piece this instance stages (LAG = 32 marks the instances for rows in pieces)
    constexpr int kPiece = (LAG == 32 && VEC) ? (R == 8 ? kTilePiece8 : kTilePiece16) : kTileMaxPiece;
    constexpr int NB = R * kPiece / (FLAT ? 4 : V) / kWave;  // accesses per lane per piece, at most
    // vectors per lane that leave in one step, at most: a row's last piece also retires the LAG columns behind it
    constexpr int NBR = (R * (kPiece + (LAG == 32 ? LAG : 0)) / 4 + kWave - 1) / kWave;
    // Rows of whole vectors in pieces: a piece is kHalves runs of 64 vectors per row, so vector b of a lane can be
    // vector lane + 64 * (b % kHalves) of row b / kHalves in every step - no index arithmetic per vector, the row and
    // the piece's time travel in scalar offsets.  (Whole rows, 75 vectors at T = 300, would need twice the memory
    // instructions that way, half of them nearly empty.)
    constexpr bool STATIC = VEC && LAG == 32;
    constexpr int kHalves = kPiece / 256;
    static_assert(!STATIC || (NB == R * kHalves && NBR == NB + R / 8), "static mapping of vectors to lanes");
    extern __shared__ __align__(16) float lds[];
    float *tile = lds;                                                    // [R][P], P = 4 (mod 32)
    uint32_t *masks = reinterpret_cast<uint32_t *>(lds + R * P);  // [R][MP]
    int *rowShift = reinterpret_cast<int *>(masks + R * MP);      // [R], used when the output is shifted
    uint32_t *cand = reinterpret_cast<uint32_t *>(rowShift + R);  // [R][MP], candidate samples (see below)
    // [R][MPT], MPT > 0: rows in pieces whose spikes are stored shifted.  A shift may reach any distance back and
    // (negative delays) forward, so the spike bits of the whole row are kept - bit LAG + t for time t - and the
    // shifted spikes of a tile's rows leave in one go after the rows' last piece.
    uint32_t *rowMasks = cand + R * MP;
    const bool record = MPT > 0;

    const int lane = threadIdx.x;
    const float amplitude = 1.0f / Ts;
    const float quiet = __builtin_nanf("");

    float tap[NU];
#pragma unroll
    for (int j = 0; j < NU; ++j) tap[j] = (j < nuSize) ? nu[j] : -0.0f;
    // this lane's taps in the candidate walk (lane p of a row: taps p, p + 64 / R, ...; -0.0f past the kernel, also
    // past NU: those samples lie in the row's padding or belong to taps that do not exist)
    float myTap[(NU + kWave / R - 1) / (kWave / R)];
#pragma unroll
    for (int j = 0; j < (NU + kWave / R - 1) / (kWave / R); ++j) {
        const int tj = lane % (kWave / R) + j * (kWave / R);
        myTap[j] = tj < nuSize ? nu[tj] : -0.0f;
    }
    // ... and for the walk over every sample, the kernel in LDS with -0.0f (whose addition changes
    // nothing) in front and behind: tapL[j] = nu[j] for j in [-(kLanesPerRow - 1), 48 - kLanesPerRow)
    constexpr int kLanesPerRow = kWave / R;
    constexpr int kAdds = (NU + kLanesPerRow - 1) / kLanesPerRow + 1;  // additions per spike and lane in that walk
    static_assert(kLanesPerRow * kAdds <= 48 - kLanesPerRow + 1, "the padded kernel in LDS");
    float *tapL = reinterpret_cast<float *>(rowMasks + R * MPT) + (kLanesPerRow - 1);
    if (lane < 48) {
        const int tj = lane - (kLanesPerRow - 1);
        tapL[tj] = (tj >= 0 && tj < nuSize) ? nu[tj] : -0.0f;
    }
    // The normal refractory kernel only lowers the potential (every tap <= 0; a NaN tap fails the test).  A sample
    // below the threshold as it arrives can then never fire, so the sequential part need only visit the samples
    // at or above it ("candidates", a few per cent): all 64 lanes mark them while the tile is staged, and the
    // walking lanes go from candidate to candidate, test the sample's current value and add the refractory
    // response in place in LDS - the same fp32 additions in the same order as the sequential loop.
    bool monotone = VEC;  // (rows of whole vectors only: elsewhere marking sample by sample costs what it saves)
    bool signedTaps = true;   // every tap negative or -0.0 (and finite): 0 * tap is then -0.0, which changes no sum
#pragma unroll
    for (int j = 0; j < NU; ++j) {
        monotone = monotone && tap[j] <= 0.0f;
        signedTaps = signedTaps && tap[j] <= 0.0f && tap[j] > -__builtin_inff() && (__builtin_bit_cast(uint32_t, tap[j]) >> 31) != 0u;
    }
    auto mark = [&](int r, int col, float x) {  // one sample
        if (x >= theta) atomicOr(cand + r * MP + (col >> 5), 1u << (col & 31));
    };
    constexpr int G = 32;               // samples per group of the window walk = bits of a spike mask

    // A "step" is one piece of one tile.  The global loads of a step are issued one step ahead
    // into x[] and stay in flight while the previous step is walked and retired.
    float x[NB * (FLAT ? 4 : V)];
    auto rows_of = [&](int64_t t) { return static_cast<int>(min(static_cast<int64_t>(R), rows - t * R)); };
    const float invT = 1.0f / static_cast<float>(T);
    auto issue = [&](int64_t t, int tL) {
        const BufferRsrc bufU = make_buffer(u + t * R * static_cast<int64_t>(T));
        if constexpr (FLAT) {  // whole rows: the tile is rows_of(t) * T / 4 consecutive vectors
            const int nVec = (rows_of(t) * T) >> 2;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const float4 q = buffer_load4(bufU, masked_offset(lane + b * kWave < nVec, (lane + b * kWave) * 16), 0);
                x[4 * b] = q.x; x[4 * b + 1] = q.y; x[4 * b + 2] = q.z; x[4 * b + 3] = q.w;
            }
            return;
        }
        const int n = min(Tc, T - tL);
        const int perRow = n / V;
        if constexpr (STATIC) {
            const int nR = rows_of(t);
            int mine[kHalves];
#pragma unroll
            for (int hf = 0; hf < kHalves; ++hf) mine[hf] = masked_offset(lane + hf * kWave < perRow, (lane + hf * kWave) * 16);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int row = b / kHalves, hf = b % kHalves;
                const float4 q = buffer_load4(bufU, row < nR ? mine[hf] : kOutOfRange, (row * T + tL) * 4);
                x[4 * b] = q.x; x[4 * b + 1] = q.y; x[4 * b + 2] = q.z; x[4 * b + 3] = q.w;
            }
            return;
        }
        const int total = rows_of(t) * perRow;
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int off = (rc.r * T + tL + rc.c * V) * 4;
            if constexpr (VEC) {
                // (masked, not skipped: a fixed number of loads lets the wait for them leave the stores that
                // are issued behind them in flight)
                const float4 q = buffer_load4(bufU, masked_offset(lane + b * kWave < total, off), 0);
                x[4 * b] = q.x; x[4 * b + 1] = q.y; x[4 * b + 2] = q.z; x[4 * b + 3] = q.w;
            } else if (lane + b * kWave < total) {
                x[b] = buffer_load(bufU, off, 0);
            }
            rc.advance(dr, dc, perRow);
        }
    };
    auto commit = [&](int64_t t, int tL) {  // tile[r][LAG + c] = u[row][tL + c]
        if constexpr (FLAT) {
            const int nVec = (rows_of(t) * T) >> 2;
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                if (lane + b * kWave < nVec) {
                    int r, c;
                    divmod_small((lane + b * kWave) << 2, T, invT, r, c);
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        tile[r * P + LAG + c] = x[4 * b + e];
                        if (monotone) mark(r, LAG + c, x[4 * b + e]);
                        if (++c == T) { c = 0; ++r; }
                    }
                }
            }
            return;
        }
        const int n = min(Tc, T - tL);
        const int perRow = n / V;
        if constexpr (STATIC) {
            const int nR = rows_of(t);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int row = b / kHalves, c = lane + (b % kHalves) * kWave;
                if (row < nR && c < perRow) {
                    *reinterpret_cast<float4 *>(tile + row * P + LAG + c * 4) = make_float4(x[4 * b], x[4 * b + 1], x[4 * b + 2], x[4 * b + 3]);
                    if (monotone) {  // (LAG and the column are multiples of 4: the four bits lie in one word; adding no bits is harmless)
                        const uint32_t bits = (x[4 * b] >= theta ? 1u : 0u) | (x[4 * b + 1] >= theta ? 2u : 0u) |
                                              (x[4 * b + 2] >= theta ? 4u : 0u) | (x[4 * b + 3] >= theta ? 8u : 0u);
                        atomicOr(cand + row * MP + ((LAG + c * 4) >> 5), bits << ((c * 4) & 31));
                    }
                }
            }
            return;
        }
        const int total = rows_of(t) * perRow;
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (lane + b * kWave < total) {
                float *dst = tile + rc.r * P + LAG + rc.c * V;
                if (VEC) {
                    *reinterpret_cast<float4 *>(dst) = make_float4(x[4 * b], x[4 * b + 1], x[4 * b + 2], x[4 * b + 3]);
                    if (monotone) {  // (the column is a multiple of 4: the four bits lie in one word)
                        const uint32_t bits = (x[4 * b] >= theta ? 1u : 0u) | (x[4 * b + 1] >= theta ? 2u : 0u) |
                                              (x[4 * b + 2] >= theta ? 4u : 0u) | (x[4 * b + 3] >= theta ? 8u : 0u);
                        const int col = LAG + rc.c * V;
                        if (bits) atomicOr(cand + rc.r * MP + (col >> 5), bits << (col & 31));
                    }
                } else {
                    *dst = x[b];
                    if (monotone) mark(rc.r, LAG + rc.c, x[b]);
                }
            }
            rc.advance(dr, dc, perRow);
        }
    };

    int64_t t = blockIdx.x;
    int tL = 0;
    if (t < tiles) issue(t, tL);
    for (int i = lane; i < R * MP; i += kWave) cand[i] = 0u;
    if (record && lane < R) rowMasks[lane * MPT + MPT - 1] = 0u;  // the word behind a row's spike bits
    wave_sync();
    if (t < tiles) commit(t, tL);
    // One trip = one step.  The next step's loads are issued first, this step's stores follow, and the next step's
    // samples are committed to LDS at the end of the same trip: loads, stores and the wait for the loads lie in one
    // straight line, so that wait can leave the younger stores in flight (their number is fixed: masked, never
    // skipped).  issue() and commit() of a step beyond the last tile do nothing.
    while (t < tiles) {
        const int nRows = rows_of(t);
        const int n = min(Tc, T - tL);  // new samples per row in this piece
        const bool last = tL + n == T;
        const int tW = tL - LAG;        // time of tile column 0 (columns [0, LAG) are carried over)
        const int64_t tn = last ? t + gridDim.x : t;  // next step: next piece of this tile, or first piece of the next
        const int tLn = last ? 0 : tL + Tc;

        wave_sync();
        // a shifted output: the rows' delays, read with the tile's first piece and ahead of the next step's loads
        // (the wait for this value then leaves those in flight)
        float rowDelay = dl.delay;
        if (dl.on && tL == 0 && dl.lut && lane < R) {
            const int64_t row = t * R + lane;
            rowDelay = dl.lut[row < rows ? (rows <= 0xffffffffLL && dl.lutSize <= 0xffffffffLL
                                                ? static_cast<int64_t>(static_cast<uint32_t>(row) % static_cast<uint32_t>(dl.lutSize))
                                                : row % dl.lutSize)
                                         : 0];
        }
        // (whole rows: one tile per work-group, nothing follows, and the walk may use the registers)
        if constexpr (LAG == 32) issue(tn, tLn);

        // ---- walk: lane = row.  Columns [0, W) become final in this step.
        const int W = last ? n + LAG : n;
        // The walking wavefront shares its SIMD's issue slots with the wavefronts that move data, so what counts
        // here is the number of instructions, not the active lanes: all 64 lanes take part, kParts = 64 / R per
        // row.  They count the row's candidates and note its non-empty candidate words together; in the walk every
        // lane of a row follows the same candidates, and on a spike each adds its own taps of the refractory
        // response (lane p: taps p, p + kParts, ...).
        constexpr int kParts = kWave / R, kRounds = (NU + kParts - 1) / kParts;
        const int cr = lane / kParts, part = lane - cr * kParts;
        bool hop = monotone;
        uint32_t nzw = 0u;   // bit w: word w of the row has candidates (at most 18 words: 512 + 32 samples)
        if (monotone) {
            int mine = 0;
            for (int w = part; w < ((W + 31) >> 5); w += kParts) {
                const uint32_t c = cand[cr * MP + w];
                mine += __builtin_popcount(c);
                nzw |= (c != 0u ? 1u : 0u) << w;
            }
#pragma unroll
            for (int off = kParts / 2; off > 0; off >>= 1) {
                mine += __shfl_xor(mine, off, kWave);
                nzw |= __shfl_xor(nzw, off, kWave);
            }
            // Going from candidate to candidate costs a round trip through LDS per visit, and the wavefront stays as long
            // as its busiest row.  Visits are spikes plus the candidates that no response has removed (below), so the
            // count of candidates on arrival only bounds them: a smooth potential that fires 4 % of the time arrives with
            // 19 % candidates (137 us this way, 156 us sample by sample, on (12,16,32,32,300)), one that fires 12 % of
            // the time with 45 % (198 us against 170 us).  Tiles with a row above the threshold half of the time or more
            // take the walk over every sample (a third: 145 us on the first of the two tensors).
            hop = __builtin_amdgcn_ballot_w64(mine * 2 > W) == 0;
        }
        const bool steady = monotone && signedTaps && !hop;
        if (hop) {
            const int words = (W + 31) >> 5;
            const uint32_t *cw = cand + cr * MP;
            uint32_t *mw = record ? rowMasks + cr * MPT + (tL >> 5) : masks + cr * MP;
            float *mine = tile + cr * P;
            for (int w = part; w < words; w += kParts) mw[w] = 0u;   // words without candidates have no spikes
            int w = 0;
            uint32_t cm = 0u, fired = 0u;
            while (__builtin_amdgcn_ballot_w64((cm | nzw) != 0u) != 0) {
                if (cm == 0u && nzw != 0u) {   // on to the row's next word with candidates
                    if (fired != 0u) mw[w] = fired;
                    fired = 0u;
                    w = __builtin_ctz(nzw);
                    nzw &= nzw - 1u;
                    cm = cw[w];
                }
                if (cm != 0u) {
                    const int k = __builtin_ctz(cm);
                    cm &= cm - 1u;
                    float *q = mine + (w << 5) + k + part;
                    // (no lane reaches past the NU samples of the response: what lies behind the row's padding
                    // belongs to the next row)
                    float val[kRounds];
#pragma unroll
                    for (int j = 0; j < kRounds; ++j)
                        if ((j + 1) * kParts <= NU || part + j * kParts < NU) val[j] = q[j * kParts];
                    const float x0 = q[-part];   // the candidate itself (one address per row: a broadcast, no shuffle)
                    if (x0 >= theta) {
                        fired |= 1u << k;
                        // The response only lowers the potential: a sample it takes below the threshold will never
                        // fire and stops being a candidate.  A potential that stays above the threshold for many
                        // samples (the output of a PSP filter) is then visited once per spike, not once per sample.
                        // Each lane knows the new value of its own samples; a ballot collects the row's verdicts
                        // (bit p of the row's field: sample k + j kParts + p), and what falls into the next word
                        // of candidates is cleared there by one lane.
                        uint64_t gone = 0u;
#pragma unroll
                        for (int j = 0; j < kRounds; ++j) {
                            const bool mineToo = (j + 1) * kParts <= NU || part + j * kParts < NU;
                            const float now = val[j] + myTap[j];
                            if (mineToo) q[j * kParts] = now;
                            const uint64_t below = __builtin_amdgcn_ballot_w64(mineToo && now < theta);
                            gone |= ((below >> (lane - part)) & ((1ull << kParts) - 1ull)) << (j * kParts);
                        }
                        gone <<= k;
                        cm &= ~static_cast<uint32_t>(gone);
                        const uint32_t over = static_cast<uint32_t>(gone >> 32);
                        if (over != 0u && part == 0 && w + 1 < words) cand[cr * MP + w + 1] &= ~over;
                    }
                }
            }
            if (fired != 0u) mw[w] = fired;
        } else {
            // Every sample in turn: 32 samples at a time pass through a register window of 32 + LAG
            // samples that is spread over the row's kParts lanes - lane p keeps the samples whose window index is
            // p (mod kParts).  The sample under test is broadcast within the row's lanes by lane-permuting moves (no
            // LDS); on a spike every lane adds the taps that fall on its own samples, kAdds instead of NU additions,
            // the same fp32 additions in the same order per sample as the sequential loop.  What counts in this
            // walk is the number of instructions (the wavefront shares its SIMD's issue slots), not the active lanes.
            constexpr int NW = (G + LAG + kParts - 1) / kParts;  // window registers per lane
            float wq[NW];                                       // wq[m] = window sample kParts m + part
            // tq[res][i] = nu[kParts i + part - res]: what a spike at a window index k = res (mod kParts) adds to
            // this lane's sample kParts (k / kParts + i) + part
            float tq[kParts][kAdds];
#pragma unroll
            for (int res = 0; res < kParts; ++res)
#pragma unroll
                for (int i = 0; i < kAdds; ++i) tq[res][i] = tapL[kParts * i + part - res];
            float *mine = tile + cr * P;
            // (the first LAG window samples: nothing before a row's start, else what the last piece left behind)
#pragma unroll
            for (int m = 0; m < NW; ++m) wq[m] = (tL == 0 || kParts * m + part >= LAG) ? quiet : mine[kParts * m + part];
            auto sample = [&](int k) {  // window sample k, from the lane of the row that keeps it
                const int in = __builtin_bit_cast(int, wq[k / kParts]);
                int q = 0;
                switch (k % 4) {  // quad_perm: the four lanes of a quad read its lane k % 4
                    case 0: q = __builtin_amdgcn_update_dpp(0, in, 0x00, 0xf, 0xf, false); break;
                    case 1: q = __builtin_amdgcn_update_dpp(0, in, 0x55, 0xf, 0xf, false); break;
                    case 2: q = __builtin_amdgcn_update_dpp(0, in, 0xaa, 0xf, 0xf, false); break;
                    default: q = __builtin_amdgcn_update_dpp(0, in, 0xff, 0xf, 0xf, false); break;
                }
                if constexpr (kParts == 8) {
                    // the quad that does not keep the sample takes it from the other one: lane i of each group of
                    // 8 reads lane 7 - i (row_half_mirror), written only in the banks (quads) that need it
                    if ((k % 8) < 4) q = __builtin_amdgcn_update_dpp(q, q, 0x141, 0xf, 0xa, false);
                    else q = __builtin_amdgcn_update_dpp(q, q, 0x141, 0xf, 0x5, false);
                }
                return __builtin_bit_cast(float, q);
            };
            uint32_t *mw = record ? rowMasks + cr * MPT + (tL >> 5) : masks + cr * MP;
            const int groups = (W + G - 1) / G;
            for (int g = 0; g < groups; ++g) {
                const int c0 = g * G;
#pragma unroll
                for (int m = LAG / kParts; m < NW; ++m) {
                    const int i = kParts * m + part;  // window index; sample c0 + i - LAG of the piece
                    if (i >= LAG && i < LAG + G) wq[m] = (c0 + i - LAG < n) ? mine[c0 + i] : quiet;
                }
                uint32_t fired = 0;
                if (steady) {
                    // a tile that is here because its rows are above the threshold most of the time: no branches - the
                    // response is added as fma(1 or 0, tap, sample), which is the addition when the sample fired and
                    // leaves every value as it is (zeros and their signs included: the taps are negative or -0.0)
                    // when it did not.  9 instructions per sample whatever happens, against 5 (nobody fires) to 14
                    // (somebody does) with the branches below.
#pragma unroll
                    for (int k = 0; k < G; ++k) {
                        const bool f = sample(k) >= theta;
                        fired |= f ? (1u << k) : 0u;
                        const float one = f ? 1.0f : 0.0f;
#pragma unroll
                        for (int i = 0; i < kAdds; ++i)
                            if (k / kParts + i < NW) wq[k / kParts + i] = __builtin_fmaf(one, tq[k % kParts][i], wq[k / kParts + i]);
                    }
                } else
#pragma unroll
                for (int k = 0; k < G; k += 2) {
                    // one scalar branch per two samples (the second sample is tested again inside, after the first
                    // one's refractory response)
                    const float xa = sample(k), xb = sample(k + 1);
                    if (__builtin_amdgcn_ballot_w64((xa >= theta) | (xb >= theta)) != 0) {
                        if (xa >= theta) {
                            fired |= 1u << k;
#pragma unroll
                            for (int i = 0; i < kAdds; ++i)
                                if (k / kParts + i < NW) wq[k / kParts + i] += tq[k % kParts][i];
                        }
                        if (sample(k + 1) >= theta) {
                            fired |= 2u << k;
#pragma unroll
                            for (int i = 0; i < kAdds; ++i)
                                if ((k + 1) / kParts + i < NW) wq[(k + 1) / kParts + i] += tq[(k + 1) % kParts][i];
                        }
                    }
                }
#pragma unroll
                for (int m = 0; m < G / kParts; ++m) mine[c0 + kParts * m + part] = wq[m];
                mw[g] = fired;  // (the same word from all lanes of the row)
#pragma unroll
                for (int m = 0; m < (LAG + kParts - 1) / kParts; ++m) wq[m] = wq[m + G / kParts];
            }
            // the LAG columns behind the final ones have taken part of the responses: back to LDS for the next piece
            if (!last) {
#pragma unroll
                for (int m = 0; m < (LAG + kParts - 1) / kParts; ++m)
                    if (kParts * m + part < LAG) mine[W + kParts * m + part] = wq[m];
            }
        }
        wave_sync();

        // ---- retire: columns [first, W) leave as u' and s, times tW + column
        {
            const BufferRsrc bufU = make_buffer(u + t * R * static_cast<int64_t>(T));
            const BufferRsrc bufS = make_buffer(s + t * R * static_cast<int64_t>(T));
            if (dl.on && tL == 0) {  // every row's shift in samples (kept for the row's further pieces)
                // (a shift of more than the longest row moves everything out, whatever its size)
                if (lane < R) rowShift[lane] = max(-(1 << 24), min(1 << 24, delay_steps(rowDelay, dl.Ts)));
                wave_sync();
            }
            // the spike bit of the sample `shift` steps before column `col` (0 outside the row)
            const int nCols = (MP - 1) << 5;
            auto bits_from = [&](int r, int col) -> uint32_t {
                const int c2 = col - rowShift[r];
                if (c2 < 0 || c2 >= nCols) return 0u;
                const int w = c2 >> 5, sh = c2 & 31;
                uint32_t m = masks[r * MP + w] >> sh;
                if (sh > 28 && w + 1 < MP - 1) m |= masks[r * MP + w + 1] << (32 - sh);
                return m;
            };
            // the same from the record of the whole row (rows in pieces): the four bits from bit c2 on
            const int nBits = T + LAG;
            auto bits_of_row = [&](int r, int c2) -> uint32_t {
                // no branches: the LDS reads of all vectors of a step go out together.  Bits before LAG and from
                // nBits on are never set, and the word behind a row's last is kept at zero.
                const bool in = c2 >= 0 && c2 < nBits;
                const int cc = in ? c2 : 0;
                const uint32_t *rm = rowMasks + r * MPT + (cc >> 5);
                const uint64_t both = (static_cast<uint64_t>(rm[1]) << 32) | rm[0];
                return in ? static_cast<uint32_t>(both >> (cc & 31)) : 0u;
            };
            if constexpr (FLAT) {
                const int nVec = (nRows * T) >> 2;
                for (int vi = lane; vi < nVec; vi += kWave) {
                    int r, c;
                    divmod_small(vi << 2, T, invT, r, c);
                    float uu[4], ss[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int col = LAG + c;   // time c of row r
                        uu[e] = tile[r * P + col];
                        const uint32_t bit = dl.on ? bits_from(r, col) : masks[r * MP + (col >> 5)] >> (col & 31);
                        ss[e] = (bit & 1u) ? amplitude : 0.0f;
                        if (++c == T) { c = 0; ++r; }
                    }
                    buffer_store4(bufU, vi * 16, 0, make_float4(uu[0], uu[1], uu[2], uu[3]));
                    buffer_store4(bufS, vi * 16, 0, make_float4(ss[0], ss[1], ss[2], ss[3]));
                }
            } else {
            const int first = (tL == 0) ? LAG : 0;  // before the first sample there is nothing to store
            const int perRow = (W - first) / V;
            const int total = nRows * perRow;
            RowCol rc;
            rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
            const int dr = kWave / perRow, dc = kWave % perRow;
            // vector b of this lane in the retire step: row, first column, and whether it exists
            auto where = [&](int b, int &r, int &col) -> bool {
                bool on;
                if constexpr (STATIC) {
                    // as in issue() and commit(); the vectors past 64 * kHalves per row (the LAG columns that a
                    // row's last piece retires as well) follow, eight per row and lane group
                    int c;
                    if (b < NB) {
                        r = b / kHalves;
                        c = lane + (b % kHalves) * kWave;
                    } else {
                        r = (b - NB) * 8 + (lane >> 3);
                        c = kHalves * kWave + (lane & 7);
                    }
                    on = r < nRows && c < perRow;
                    col = first + c * 4;
                } else {
                    on = lane + b * kWave < total;
                    r = rc.r;
                    col = first + rc.c * V;
                    rc.advance(dr, dc, perRow);
                }
                if (!on) {
                    r = 0;
                    col = first;
                }
                return on;
            };
            if constexpr (VEC) {
              if (!dl.on) {
                // a fixed number of (masked) stores, see above.  Half of a step's vectors at a time: their LDS reads
                // go out together, the stores follow (one read-wait-store chain per vector cost a third of a step)
                constexpr int HB = (NBR + 1) / 2;
#pragma unroll
                for (int b0 = 0; b0 < NBR; b0 += HB) {
                    float4 uu[HB];
                    uint32_t word[HB];
                    int offs[HB], sh[HB];
#pragma unroll
                    for (int i = 0; i < HB; ++i) {
                        if (b0 + i < NBR) {
                            int r, col;
                            const bool on = where(b0 + i, r, col);
                            uu[i] = *reinterpret_cast<const float4 *>(tile + r * P + col);
                            word[i] = masks[r * MP + (col >> 5)];
                            sh[i] = col & 31;
                            offs[i] = masked_offset(on, (r * T + tW + col) * 4);
                        }
                    }
#pragma unroll
                    for (int i = 0; i < HB; ++i) {
                        if (b0 + i < NBR) {
                            const uint32_t m = word[i] >> sh[i];
                            buffer_store4(bufU, offs[i], 0, uu[i]);
                            buffer_store4(bufS, offs[i], 0,
                                          make_float4((m & 1u) ? amplitude : 0.0f, (m & 2u) ? amplitude : 0.0f,
                                                      (m & 4u) ? amplitude : 0.0f, (m & 8u) ? amplitude : 0.0f));
                        }
                    }
                }
              } else {
#pragma unroll
                for (int b = 0; b < NBR; ++b) {
                    int r, col;
                    const bool on = where(b, r, col);
                    const float *src = tile + r * P + col;
                    // rows in pieces with a shifted output: a shift towards later times only needs spikes that are
                    // final by now; the rows with a negative shift wait for their last piece
                    const int shift = record ? rowShift[r] : 0;
                    const uint32_t m = record ? bits_of_row(r, tL + col - shift)
                                              : dl.on ? bits_from(r, col) : masks[r * MP + (col >> 5)] >> (col & 31);
                    const int off = masked_offset(on, (r * T + tW + col) * 4);
                    buffer_store4(bufU, off, 0, *reinterpret_cast<const float4 *>(src));
                    buffer_store4(bufS, shift < 0 ? kOutOfRange : off, 0,
                                  make_float4((m & 1u) ? amplitude : 0.0f, (m & 2u) ? amplitude : 0.0f,
                                              (m & 4u) ? amplitude : 0.0f, (m & 8u) ? amplitude : 0.0f));
                }
              }
            } else {
#pragma unroll 4
                for (int g0 = lane; g0 < total; g0 += kWave) {
                    const int col = first + rc.c * V;
                    const int off = (rc.r * T + tW + col) * 4;
                    const float *src = tile + rc.r * P + col;
                    const uint32_t m = dl.on ? bits_from(rc.r, col) : masks[rc.r * MP + (col >> 5)] >> (col & 31);
                    buffer_store(bufU, off, 0, src[0]);
                    buffer_store(bufS, off, 0, (m & 1u) ? amplitude : 0.0f);
                    rc.advance(dr, dc, perRow);
                }
            }
            }
        }
        wave_sync();

        if constexpr (VEC) {
            bool early = false;  // a row of this tile takes its spikes from later times
            if (record && last) early = __builtin_amdgcn_ballot_w64(lane < nRows && rowShift[lane < R ? lane : 0] < 0) != 0;
            if (early) {
                // the rows are complete: the spikes of those rows, shifted, from the record of the whole row
                const BufferRsrc bufS = make_buffer(s + t * R * static_cast<int64_t>(T));
                const int nBits = T + LAG, nWords = (nBits + 31) >> 5;
                const int perRow = T >> 2;
                const int total = nRows * perRow;
                RowCol rc;
                rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
                const int dr = kWave / perRow, dc = kWave % perRow;
                for (int g0 = lane; g0 < total; g0 += kWave, rc.advance(dr, dc, perRow)) {
                    if (rowShift[rc.r] >= 0) continue;
                    const int c2 = LAG + 4 * rc.c - rowShift[rc.r];
                    uint32_t m = 0u;
                    if (c2 > -4 && c2 < nBits) {
                        // (bits before LAG and from nBits on are never set; c2 may be up to 3 below zero)
                        const int w = c2 >> 5, sh = c2 & 31;
                        const uint32_t *rm = rowMasks + rc.r * MPT;
                        if (c2 >= 0) {
                            m = rm[w] >> sh;
                            if (sh > 28 && w + 1 < nWords) m |= rm[w + 1] << (32 - sh);
                        } else {
                            m = rm[0] << -c2;
                        }
                    }
                    buffer_store4(bufS, (rc.r * T + 4 * rc.c) * 4, 0,
                                  make_float4((m & 1u) ? amplitude : 0.0f, (m & 2u) ? amplitude : 0.0f,
                                              (m & 4u) ? amplitude : 0.0f, (m & 8u) ? amplitude : 0.0f));
                }
                wave_sync();
            }
        }
        // rows in pieces: the LAG columns behind this piece's final ones, and their candidates, open the next
        // piece (LAG is one word of candidates then); every other word of candidates starts empty
        if (!last) {
            for (int i = lane; i < R * (LAG / 4); i += kWave) {
                const int r = i / (LAG / 4), c4 = i - r * (LAG / 4);
                *reinterpret_cast<float4 *>(tile + r * P + 4 * c4) = *reinterpret_cast<const float4 *>(tile + r * P + n + 4 * c4);
            }
            if (lane < R) cand[lane * MP] = cand[lane * MP + (n >> 5)];
            wave_sync();
        }
        for (int i = lane; i < R * MP; i += kWave)
            if (last || i % MP != 0) cand[i] = 0u;
        wave_sync();
        if constexpr (LAG == 32) commit(tn, tLn);
        else if (tn < tiles) {  // (not reached: whole rows are launched with one work-group per tile)
            issue(tn, tLn);
            commit(tn, tLn);
        }
        t = tn;
        tL = tLn;
    }
}

// ---- surrogate gradient ------------------------------------------------------------------------------
// One pass over three tensors (12 B per neuron-timestep), shaped like the fastest copy this GPU
// runs: one 16-byte vector per lane, one pass per work-group, streaming cache policy.
typedef float vec4f __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void spike_bwd_vec_kernel(float *gradIn, const float *gradOut,
                                                            const float *__restrict__ u, float theta,
                                                            float tau, float gain, int64_t quads)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= quads) return;
    const vec4f g = __builtin_nontemporal_load(reinterpret_cast<const vec4f *>(gradOut) + i);
    const vec4f x = __builtin_nontemporal_load(reinterpret_cast<const vec4f *>(u) + i);
    vec4f o;
    o.x = g.x * spike_pdf(x.x, theta, tau, gain);
    o.y = g.y * spike_pdf(x.y, theta, tau, gain);
    o.z = g.z * spike_pdf(x.z, theta, tau, gain);
    o.w = g.w * spike_pdf(x.w, theta, tau, gain);
    __builtin_nontemporal_store(o, reinterpret_cast<vec4f *>(gradIn) + i);
}

// The same gradient behind a shifted output: with s_out[t] = spike[t - k] the gradient that reaches
// the spike at time t is gradOut[t + k].  One lane per VEC output samples; the row's shift comes from
// the per-neuron table or the one delay, like in the forward pass.
template <int VEC>
__global__ __launch_bounds__(256) void spike_bwd_delayed_kernel(float *gradIn, const float *gradOut,
                                                                const float *__restrict__ u, SpikeDelay dl,
                                                                int T, FastDiv byTV, float theta, float tau,
                                                                float gain, int64_t vectors)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i >= vectors) return;
    // rows are addressed relative to the work-group's first row so that offsets stay 32 bit
    const int64_t first = static_cast<int64_t>(blockIdx.x) * 256;
    const int64_t row0 = first / byTV.d;
    const uint32_t local = static_cast<uint32_t>(i - row0 * byTV.d);
    const uint32_t rl = fastdiv(local, byTV);
    const int t = static_cast<int>(local - rl * byTV.d) * VEC;
    const int64_t row = row0 + rl;
    const int k = delay_steps(dl.lut ? dl.lut[row % dl.lutSize] : dl.delay, dl.Ts);
    const BufferRsrc gB = make_buffer(gradOut + row0 * T);
    const int rowBytes = static_cast<int>(rl) * T * 4;
    float g[VEC], x[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
        // t + k + e computed without overflow for any k
        const int64_t src = static_cast<int64_t>(t) + k + e;
        g[e] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(
            gB, masked_offset(src >= 0 && src < T, rowBytes + static_cast<int>(src < T && src >= 0 ? src : 0) * 4), 0, 0));
        x[e] = u[row * T + t + e];
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) gradIn[row * T + t + e] = g[e] * spike_pdf(x[e], theta, tau, gain);
}

__global__ __launch_bounds__(256) void spike_bwd_scalar_kernel(float *gradIn, const float *gradOut,
                                                               const float *__restrict__ u, float theta,
                                                               float tau, float gain, int64_t numel)
{
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < numel) gradIn[i] = gradOut[i] * spike_pdf(u[i], theta, tau, gain);
}

}  // namespace slayer

namespace slayer {

// Picks and launches the spike kernel.  With a shift of the output (dl.on) only the tile kernel with
// whole rows qualifies; other shapes return SLAYER_EUNSUPPORTED before anything is launched.
static int launch_get_spikes(float *s, float *u, const float *nu, int64_t nNeurons, int64_t T, int64_t nuSize,
                             float theta, float Ts, hipStream_t st, const SpikeDelay &dl)
{

    const int64_t groups = ceil_div(nNeurons, kWave);
    const bool stream_ok = !generic_forced() && T < (1LL << 30) && groups < (1LL << 31);
    const bool window_ok = stream_ok && T <= kBufferMaxT;
#define SLAYER_SPIKE_TILE_LAUNCH(NU, LAGV, RV)                                                           \
    do {                                                                                                \
        if (vec)                                                                                        \
            hipLaunchKernelGGL((spike_tile_kernel<NU, kTileVec, LAGV, RV>), dim3(grid), dim3(kWave),    \
                               lds, st, s, u, nu, nNeurons, static_cast<int>(T),                        \
                               static_cast<int>(nuSize), Tc, P, MP, MPT, tiles, theta, Ts, dl);         \
        else if (flat && RV == 8)                                                                       \
            hipLaunchKernelGGL((spike_tile_kernel<NU, (RV == 8 ? kTileFlat : kTileScalar), LAGV, RV>),  \
                               dim3(grid), dim3(kWave), lds, st, s, u, nu, nNeurons,                    \
                               static_cast<int>(T), static_cast<int>(nuSize), Tc, P, MP, MPT, tiles,    \
                               theta, Ts, dl);                                                          \
        else                                                                                            \
            hipLaunchKernelGGL((spike_tile_kernel<NU, kTileScalar, LAGV, RV>), dim3(grid), dim3(kWave), \
                               lds, st, s, u, nu, nNeurons, static_cast<int>(T),                        \
                               static_cast<int>(nuSize), Tc, P, MP, MPT, tiles, theta, Ts, dl);         \
        return launch_status();                                                                         \
    } while (0)
#define SLAYER_SPIKE_TILE_LAG(NU, LAGV)                                                                  \
    do {                                                                                                \
        /* Rows that travel whole: 8-row tiles, one work-group per tile - many short-lived groups per   \
           CU overlap the memory phases of some with the walks of others better than a loop does.       \
           Rows in pieces: the group loops over the pieces; 16 rows per tile and pieces of 256 samples  \
           unless that would leave wavefront slots of the GPU empty: then 8 rows and, for rows of whole \
           vectors, pieces of 512 samples, which doubles the bytes in flight per wavefront. */          \
        int Tc = whole ? static_cast<int>(T) : kTilePiece16;                                            \
        int cols, P, MP;                                                                                \
        auto layout = [&]() {                                                                           \
            cols = (LAGV + Tc + 31) & ~31; /* the walk goes in groups of 32 columns */                  \
            /* 4 (mod 8): rows are 16-byte aligned and 8 of them start in different banks; a refractory \
               response that is added in place may reach NU - 1 columns past the last one */           \
            P = cols + 4;                                                                               \
            while (P - (LAGV + Tc) < NU - 1) P += 8;                                                    \
            MP = cols / 32 + 1;                                                                         \
        };                                                                                              \
        layout();                                                                                       \
        const int64_t slots16 = static_cast<int64_t>(cus) * (160 * 1024 / ((16LL * P + 32 * MP + 16) * 4)); \
        const int rowsPerTile = (!whole && ceil_div(nNeurons, 16) >= slots16) ? 16 : 8;                 \
        if (!whole && rowsPerTile == 8 && vec) {                                                        \
            Tc = kTilePiece8;                                                                           \
            layout();                                                                                   \
        }                                                                                               \
        /* shifted spikes of rows in pieces: the spike bits of whole rows stay in LDS */                \
        const int MPT = (dl.on && !whole) ? static_cast<int>((T + LAGV + 31) / 32 + 1) : 0;             \
        auto lds_bytes = [&]() {                                                                        \
            /* tile, spike and candidate bits, row shifts, whole rows' spike bits, the padded kernel */  \
            return (static_cast<size_t>(rowsPerTile) * P + 2 * rowsPerTile * MP + rowsPerTile +         \
                    static_cast<size_t>(rowsPerTile) * MPT + 48) * sizeof(float);                       \
        };                                                                                              \
        /* eight wavefronts per compute unit are what the 8-row tiles of a small tensor need to be      \
           resident all at once: shorter pieces if the tile does not fit an eighth of the LDS */        \
        while (!whole && rowsPerTile == 8 && vec && Tc > kTilePiece16 && lds_bytes() > 160 * 1024 / 8) { \
            Tc -= 32;                                                                                   \
            layout();                                                                                   \
        }                                                                                               \
        const size_t lds = lds_bytes();                                                                 \
        const int64_t tiles = ceil_div(nNeurons, rowsPerTile);                                          \
        const int64_t resident = static_cast<int64_t>(cus) * (160 * 1024 / static_cast<int64_t>(lds));  \
        if (tiles >= (1LL << 31)) return SLAYER_EUNSUPPORTED;                                           \
        const unsigned grid = static_cast<unsigned>((whole || tiles < resident) ? tiles : resident);    \
        if (rowsPerTile == 16) SLAYER_SPIKE_TILE_LAUNCH(NU, LAGV, 16);                                  \
        SLAYER_SPIKE_TILE_LAUNCH(NU, LAGV, 8);                                                          \
    } while (0)
#define SLAYER_SPIKE_TILE(NU)                                                                            \
    do {                                                                                                \
        if (whole) SLAYER_SPIKE_TILE_LAG(NU, ((NU + 2) & ~3));                                          \
        SLAYER_SPIKE_TILE_LAG(NU, 32);                                                                  \
    } while (0)
    // a shifted output: rows that travel whole, or rows of whole vectors whose spike bits fit into LDS
    if (dl.on && !(window_ok && nuSize <= 24 &&
                   (T <= kTileMaxPiece || (T <= kSpikeRecordMaxT && T % 4 == 0 && aligned16(s) && aligned16(u)))))
        return SLAYER_EUNSUPPORTED;
    if (window_ok && nuSize <= 24) {
        // short rows travel whole; long rows in pieces
        const bool whole = T <= kTileMaxPiece;
        const bool vec = (T % 4 == 0) && aligned16(s) && aligned16(u);
        // whole rows that are not whole vectors, in a tensor that is: 8-row tiles are aligned runs
        const bool flat = whole && !vec && T >= 4 && (nNeurons * T) % 4 == 0 && aligned16(s) && aligned16(u);
        const int cus = compute_units();
        if (nuSize <= 4) SLAYER_SPIKE_TILE(4);
        if (nuSize <= 8) SLAYER_SPIKE_TILE(8);
        if (nuSize <= 12) SLAYER_SPIKE_TILE(12);
        if (nuSize <= 16) SLAYER_SPIKE_TILE(16);
        SLAYER_SPIKE_TILE(24);
    }
#undef SLAYER_SPIKE_TILE
#undef SLAYER_SPIKE_TILE_LAG
#undef SLAYER_SPIKE_TILE_LAUNCH
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

}  // namespace slayer

extern "C" int slayer_get_spikes_f32(float *s, float *u, const float *nu, int64_t nNeurons,
                                     int64_t T, int64_t nuSize, float theta, float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || nuSize < 0) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !u || (nuSize > 0 && !nu)) return SLAYER_EINVAL;
    return launch_get_spikes(s, u, nu, nNeurons, T, nuSize, theta, Ts, static_cast<hipStream_t>(stream),
                             SpikeDelay{nullptr, 0, 0.0f, 1.0f, 0});
}

extern "C" int slayer_get_spikes_delayed_f32(float *s, float *u, const float *nu, const float *delayLut,
                                             int64_t lutSize, float delay, float delayTs, int64_t nNeurons,
                                             int64_t T, int64_t nuSize, float theta, float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || nuSize < 0 || lutSize < 0) return SLAYER_EINVAL;
    if (delayLut && (lutSize == 0 || nNeurons % lutSize != 0)) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !u || (nuSize > 0 && !nu)) return SLAYER_EINVAL;
    return launch_get_spikes(s, u, nu, nNeurons, T, nuSize, theta, Ts, static_cast<hipStream_t>(stream),
                             SpikeDelay{delayLut, lutSize, delay, delayTs, 1});
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
    const int64_t lanes = vec4 ? numel / 4 : numel;
    const int64_t blocks = ceil_div(lanes, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    if (vec4)
        hipLaunchKernelGGL(spike_bwd_vec_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           gradIn, gradOut, u, theta, tau, gain, lanes);
    else
        hipLaunchKernelGGL(spike_bwd_scalar_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st,
                           gradIn, gradOut, u, theta, tau, gain, lanes);
    return launch_status();
}

extern "C" int slayer_spike_bwd_delayed_f32(float *gradIn, const float *gradOut, const float *u,
                                            const float *delayLut, int64_t lutSize, float delay, float delayTs,
                                            int64_t nNeurons, int64_t T, float theta, float tau, float scale,
                                            void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || lutSize < 0) return SLAYER_EINVAL;
    if (delayLut && (lutSize == 0 || nNeurons % lutSize != 0)) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!gradIn || !gradOut || !u) return SLAYER_EINVAL;
    if (T > kBufferMaxT) return SLAYER_EUNSUPPORTED;  // 256 vectors of a work-group must stay below 2 GiB
    const SpikeDelay dl{delayLut, lutSize, delay, delayTs, 1};
    const bool vec = T % 4 == 0;
    const int64_t vectors = nNeurons * (vec ? T / 4 : T);
    const int64_t blocks = ceil_div(vectors, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const FastDiv byTV = make_fastdiv(static_cast<uint32_t>(vec ? T / 4 : T));
    if (vec)
        hipLaunchKernelGGL(spike_bwd_delayed_kernel<4>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, gradIn,
                           gradOut, u, dl, static_cast<int>(T), byTV, theta, tau, scale / tau, vectors);
    else
        hipLaunchKernelGGL(spike_bwd_delayed_kernel<1>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, gradIn,
                           gradOut, u, dl, static_cast<int>(T), byTV, theta, tau, scale / tau, vectors);
    return launch_status();
}

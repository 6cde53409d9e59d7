// Loihi CUBA neuron: int32 current/voltage with sign-magnitude decay (>>12), integer
// threshold, refractory delay.  Sequential in time per neuron, parallel over neurons.
//
// HBM-bound (16 B per neuron-timestep: read w, write spike, voltage, current).  Same row-tile
// scheme as the SRM spike kernel: a 64-lane work-group owns 16 consecutive rows and moves them
// through LDS in pieces of up to 128 samples per row, so global memory is read and written as
// contiguous runs with 16-byte accesses; lanes 0..15 then update their row sequentially, 32
// samples at a time from registers.  The neuron state (current, voltage, refractory countdown)
// stays in registers across pieces.  The piece's input tile is overwritten in place by the
// current; the voltage has its own tile; spikes travel as 32-bit masks.  Work-groups are
// persistent and issue the loads of the next piece before updating the current one.
//
// Refractory bookkeeping: the sequential formulation keeps a counter that is incremented at a
// spike and decremented refDelay steps later by re-reading the spike it wrote then.  Because a
// spike needs the counter to be zero, the counter only takes the values 0 and 1, and "1" lasts
// exactly until refDelay steps after the spike.  A countdown register set to refDelay at a
// spike and decremented once per step (before the threshold test) is therefore the same
// automaton, without the read-back.
#include "common.h"

#ifndef LOIHI_ROWS
#define LOIHI_ROWS 32
#define LOIHI_LPP 1
#endif
#define LOIHI_PIECE 64

namespace slayer {


// The update below is written without branches: one time step is about 30 vector instructions.

// float -> int32 the way the hardware converts: toward zero, saturating, NaN -> 0
// (v_cvt_i32_f32; a C cast would be undefined for the out-of-range inputs).
__device__ __forceinline__ int cvt_trunc_sat(float x)
{
    int r;
    asm("v_cvt_i32_f32 %0, %1" : "=v"(r) : "v"(x));
    return r;
}

// sign(x) * ((|x| * keep) >> 12) in 32-bit wrap-around arithmetic, keep = 4096 - decay
__device__ __forceinline__ uint32_t loihi_decay(int x, uint32_t keep)
{
    const uint32_t sgn = static_cast<uint32_t>(x >> 31);           // 0 or 0xFFFFFFFF
    const uint32_t mag = (static_cast<uint32_t>(x) ^ sgn) - sgn;    // |x| (2^31 stays 2^31)
    const uint32_t scaled = (mag * keep) >> 12;
    return (scaled ^ sgn) - sgn;                                    // negated again when x < 0
}

struct LoihiState {
    int current;
    int voltage;
    int countdown;  // steps until the neuron may spike again (0 = not refractory)
};

struct LoihiParams {
    uint32_t weightShift, keepI, keepV, vDecay;
    int refDelay, theta;
    int delay;  // the spike output is written `delay` samples late (0..31), zeros before: a fused delayShift
};

// The spike bits of 32 consecutive samples, delayed by p.delay samples: the bits that leave at
// the top come back at the bottom of the next group of the same row (prev = the previous group's
// undelayed bits, 0 at the start of a row).
__device__ __forceinline__ uint32_t loihi_delayed(uint32_t fired, uint32_t prev, int delay)
{
    return delay ? ((fired << delay) | (prev >> (32 - delay))) : fired;
}

// One time step (t >= 1).  Returns the spike (0/1); cOut / vOut are the reported current / voltage.
__device__ __forceinline__ uint32_t loihi_step(LoihiState &st, const LoihiParams &p, float w,
                                               float &cOut, float &vOut)
{
    const uint32_t wi = static_cast<uint32_t>(cvt_trunc_sat(w));
    const int cNew = static_cast<int>(loihi_decay(st.current, p.keepI) + (wi << p.weightShift));
    const int vNew = static_cast<int>(loihi_decay(st.voltage, p.keepV) + static_cast<uint32_t>(cNew));
    const int cd = max(st.countdown - 1, 0);
    const bool quiet = cd == 0;                       // not refractory at this step
    const bool spike = quiet & (vNew > p.theta);
    st.voltage = (quiet & !spike) ? vNew : 0;
    st.countdown = spike ? p.refDelay : cd;
    st.current = cNew;
    cOut = static_cast<float>(cNew);
    vOut = spike ? static_cast<float>(static_cast<int>(p.vDecay)) : static_cast<float>(st.voltage);
    return spike ? 1u : 0u;
}

// The same step for states of small magnitude, at about two thirds of the cost (a 32-bit integer
// multiplication takes four times as long as the other instructions here, a 24-bit one does not).
// For |x| * keep < 2^31 nothing wraps around and sign * ((|x| * keep) >> 12) is x * keep / 4096
// rounded toward zero = (x * keep + (x < 0 ? 4095 : 0)) >> 12 with an arithmetic shift.  Valid while
// keep <= 4096 and both states stay inside (-kLoihiSmall, kLoihiSmall); lo / hi collect the extremes
// of the new current and voltage so that the caller can check that afterwards: a value is
// computed correctly whenever the previous state was in range, so the first value that leaves the
// range is itself correct and is seen.
constexpr int kLoihiSmall = 1 << 19;

__device__ __forceinline__ int loihi_decay_small(int x, int keep)
{
    int scaled;  // x * keep + bias from the low 24 bits of x and keep (the compiler's own choice for
                 // __mul24 plus an addition is a 64-bit multiply-add, as slow as the 32-bit multiplication)
    asm("v_mad_i32_i24 %0, %1, %2, %3" : "=v"(scaled) : "v"(x), "v"(keep), "v"((x >> 31) & 4095));
    return scaled >> 12;
}

__device__ __forceinline__ uint32_t loihi_step_small(LoihiState &st, const LoihiParams &p, float w,
                                                     float &cOut, float &vOut, int &lo, int &hi)
{
    const uint32_t wi = static_cast<uint32_t>(cvt_trunc_sat(w));
    const int cNew = static_cast<int>(static_cast<uint32_t>(loihi_decay_small(st.current, static_cast<int>(p.keepI))) +
                                      (wi << p.weightShift));
    const int vNew = static_cast<int>(static_cast<uint32_t>(loihi_decay_small(st.voltage, static_cast<int>(p.keepV))) +
                                      static_cast<uint32_t>(cNew));
    lo = min(min(lo, cNew), vNew);
    hi = max(max(hi, cNew), vNew);
    const int cd = max(st.countdown - 1, 0);
    const bool quiet = cd == 0;
    const bool spike = quiet & (vNew > p.theta);
    st.voltage = (quiet & !spike) ? vNew : 0;
    st.countdown = spike ? p.refDelay : cd;
    st.current = cNew;
    cOut = static_cast<float>(cNew);
    vOut = spike ? static_cast<float>(static_cast<int>(p.vDecay)) : static_cast<float>(st.voltage);
    return spike ? 1u : 0u;
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
    LoihiState st = {0, 0, 0};
    uint32_t history = 0;  // bit k: the spike k samples ago
    s[base] = 0.0f;
    if (v) v[base] = 0.0f;
    if (u) u[base] = 0.0f;
    for (int64_t t = 1; t < T; ++t) {
        float c, vo;
        history = (history << 1) | loihi_step(st, p, w[base + t], c, vo);
        s[base + t] = static_cast<float>((history >> p.delay) & 1u);
        if (u) u[base + t] = c;
        if (v) v[base + t] = vo;
    }
}

// ---- row-tile kernel ---------------------------------------------------------------------------------
// R rows per tile (= lanes that update), PIECE = samples per row and piece at most.
template <bool VEC, int R, int PIECE>
__global__ __launch_bounds__(64) void loihi_tile_kernel(float *__restrict__ s, float *__restrict__ v,
                                                        float *__restrict__ u, const float *__restrict__ w,
                                                        int64_t rows, int T, int Tc, int P, int MP,
                                                        int64_t tiles, LoihiParams p)
{
    constexpr int G = 32;           // samples per update group = bits of a spike mask
    constexpr int V = VEC ? 4 : 1;  // samples per global access
    constexpr int NB = R * PIECE / V / kWave;  // accesses per lane per piece, at most
    extern __shared__ __align__(16) float lds[];
    float *tileC = lds;                    // [R][P]: input, then current;  P = 4 (mod 32)
    float *tileV = lds + R * P;   // [R][P]: voltage
    uint32_t *masks = reinterpret_cast<uint32_t *>(lds + 2 * R * P);  // [R][MP]

    const int lane = threadIdx.x;
    LoihiState st = {0, 0, 0};
    uint32_t prevFired = 0;

    float x[NB * V];
    auto rows_of = [&](int64_t t) { return static_cast<int>(min(static_cast<int64_t>(R), rows - t * R)); };
    auto issue = [&](int64_t t, int tL) {
        const BufferRsrc bufW = make_buffer(w + t * R * static_cast<int64_t>(T));
        const int perRow = min(Tc, T - tL) / V;
        const int total = rows_of(t) * perRow;
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (lane + b * kWave < total) {
                const int off = (rc.r * T + tL + rc.c * V) * 4;
                if (VEC) {
                    const float4 q = buffer_load4<kCached>(bufW, off, 0);
                    x[4 * b] = q.x; x[4 * b + 1] = q.y; x[4 * b + 2] = q.z; x[4 * b + 3] = q.w;
                } else {
                    x[b] = buffer_load<kCached>(bufW, off, 0);
                }
            }
            rc.advance(dr, dc, perRow);
        }
    };
    auto commit = [&](int64_t t, int tL) {
        const int perRow = min(Tc, T - tL) / V;
        const int total = rows_of(t) * perRow;
        RowCol rc;
        rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
        const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (lane + b * kWave < total) {
                float *dst = tileC + rc.r * P + rc.c * V;
                if (VEC) *reinterpret_cast<float4 *>(dst) = make_float4(x[4 * b], x[4 * b + 1], x[4 * b + 2], x[4 * b + 3]);
                else *dst = x[b];
            }
            rc.advance(dr, dc, perRow);
        }
    };

    int64_t t = blockIdx.x;
    int tL = 0;
    if (t < tiles) issue(t, tL);
    while (t < tiles) {
        const int nRows = rows_of(t);
        const int n = min(Tc, T - tL);
        const bool last = tL + n == T;

        commit(t, tL);
        wave_sync();
        {
            const int64_t tn = last ? t + gridDim.x : t;
            const int tLn = last ? 0 : tL + Tc;
            if (tn < tiles) issue(tn, tLn);
        }

        // ---- sequential update: lane = row
        if (lane < R) {
            if (tL == 0) { st = {0, 0, 0}; prevFired = 0; }
            float *mineC = tileC + lane * P;
            float *mineV = tileV + lane * P;
            const int groups = (n + G - 1) / G;
            for (int g = 0; g < groups; ++g) {
                const int c0 = g * G;
                float in[G], cur[G], vol[G];
#pragma unroll
                for (int k = 0; k < G; k += 4) {
                    const float4 q = *reinterpret_cast<const float4 *>(mineC + c0 + k);
                    in[k] = q.x; in[k + 1] = q.y; in[k + 2] = q.z; in[k + 3] = q.w;
                }
                uint32_t fired = 0;
#pragma unroll
                for (int k = 0; k < G; ++k) {
                    if (tL + c0 + k == 0) {  // t = 0 is forced to zero and leaves the state untouched
                        cur[k] = 0.0f;
                        vol[k] = 0.0f;
                    } else {
                        fired |= loihi_step(st, p, in[k], cur[k], vol[k]) << k;
                    }
                }
#pragma unroll
                for (int k = 0; k < G; k += 4) {
                    *reinterpret_cast<float4 *>(mineC + c0 + k) = make_float4(cur[k], cur[k + 1], cur[k + 2], cur[k + 3]);
                    *reinterpret_cast<float4 *>(mineV + c0 + k) = make_float4(vol[k], vol[k + 1], vol[k + 2], vol[k + 3]);
                }
                masks[lane * MP + g] = loihi_delayed(fired, prevFired, p.delay);
                prevFired = fired;
            }
        }
        wave_sync();

        // ---- retire (voltage and current only when the caller wants them)
        {
            const int64_t base = t * R * static_cast<int64_t>(T);
            const BufferRsrc bufS = make_buffer(s + base);
            const BufferRsrc bufV = make_buffer((v ? v : s) + base);
            const BufferRsrc bufU = make_buffer((u ? u : s) + base);
            const int perRow = n / V;
            const int total = nRows * perRow;
            RowCol rc;
            rc.init(lane, perRow, 1.0f / static_cast<float>(perRow));
            const int dr = kWave / perRow, dc = kWave % perRow;
#pragma unroll 4
            for (int g0 = lane; g0 < total; g0 += kWave) {
                const int col = rc.c * V;
                const int off = (rc.r * T + tL + col) * 4;
                const uint32_t m = masks[rc.r * MP + (col >> 5)] >> (col & 31);
                if (VEC) {
                    if (u) buffer_store4(bufU, off, 0, *reinterpret_cast<const float4 *>(tileC + rc.r * P + col));
                    if (v) buffer_store4(bufV, off, 0, *reinterpret_cast<const float4 *>(tileV + rc.r * P + col));
                    buffer_store4(bufS, off, 0,
                                  make_float4((m & 1u) ? 1.0f : 0.0f, (m & 2u) ? 1.0f : 0.0f,
                                              (m & 4u) ? 1.0f : 0.0f, (m & 8u) ? 1.0f : 0.0f));
                } else {
                    if (u) buffer_store(bufU, off, 0, tileC[rc.r * P + col]);
                    if (v) buffer_store(bufV, off, 0, tileV[rc.r * P + col]);
                    buffer_store(bufS, off, 0, (m & 1u) ? 1.0f : 0.0f);
                }
                rc.advance(dr, dc, perRow);
            }
        }
        wave_sync();

        if (last) { t += gridDim.x; tL = 0; }
        else tL += Tc;
    }
}

// ---- line-aligned row-tile kernel ---------------------------------------------------------------------
// Same scheme, for rows that are whole 16-byte vectors, with one refinement that matters a lot on
// HBM: every piece of every row is a whole number of 128-byte memory lines.  Row r does not cut
// its samples at multiples of the piece length but at the 128-byte boundaries of its own
// storage: with o_r = (address of the row's first sample mod 128) / 4, piece j of row r holds the
// samples [32 LPP j - o_r, 32 LPP (j+1) - o_r).  Lanes are independent in the sequential update,
// so it does not matter that they are at slightly different times.  All four tensors are then
// read and written as full, aligned lines (except at the two ends of a row); pieces that start
// or end in the middle of a line make the memory system write that line twice, partially, which
// measured about three times slower for the three output tensors.
//
// MERGE (needs LPP = 1 and rows of at least 64 samples): the memory line in which row r ends is
// also the line in which row r+1 begins.  Stored by both rows it would be written twice,
// partially, ten pieces apart.  Instead row r+1 keeps the results of its first line in
// registers and hands them over when row r reaches that line, so that it goes out once, whole.
// Only the first and the last row of a tile still write a partial line.
// R rows per tile (= lanes that update), LPP = 128-byte lines per row and piece.
//
// ELEM (with MERGE): rows that are not whole 16-byte vectors (T % 4 != 0) in tensors that are
// (16-byte aligned, rows * T % 4 == 0).  Lines and vectors are cut from memory, not from rows, so
// all accesses stay aligned; what changes is that the vector in which a row ends can also hold
// the first samples of the next row.  Loads simply fetch such a vector for both rows, and the
// hand-over of a row's first line to the row above works sample by sample.  R * T * 4 is a
// multiple of 128 for R = 32 or 64, so a tile still begins and ends on a line boundary.
//
// OUTS: 0 = the pointers say which outputs are wanted; 2 = spikes and voltage (u is null), 1 = spikes
// alone (v and u are null), known at compile time so that the unwanted results cost neither
// instructions nor registers, nor (the voltage tile of OUTS = 1) shared memory.
template <int R, int LPP, bool MERGE, bool ELEM = false, int OUTS = 0>
__global__ __launch_bounds__(64, 2) void loihi_lines_kernel(float *__restrict__ s, float *__restrict__ v,
                                                         float *__restrict__ u, const float *__restrict__ w,
                                                         int64_t rows, int T, int64_t tiles, LoihiParams p)
{
    constexpr int G = 32;              // samples per line = samples per update group = bits of a mask
    constexpr int TC = G * LPP;        // samples per row and piece
    constexpr int QP = TC / 4;         // 16-byte vectors per row and piece
    constexpr int RPI = kWave / QP;    // rows covered by one wave-wide access
    constexpr int NB = R / RPI;        // accesses per lane per piece
    constexpr int P = TC + 4;          // LDS pitch = 4 (mod 32): 16-byte aligned rows in different banks
    constexpr bool kCur = OUTS == 0, kVol = OUTS != 1;  // results that may be wanted at all
    __shared__ __align__(16) float tileC[R * P];  // input, then current
    __shared__ __align__(16) float tileV[kVol ? R * P : 4];  // voltage
    __shared__ uint32_t masks[R * LPP];
    if (OUTS != 0) u = nullptr;
    if (OUTS == 1) v = nullptr;

    const int lane = threadIdx.x;
    const int subRow = lane / QP;         // row within an access
    const int col = (lane % QP) * 4;      // first column of this lane's vector
    const int pieces = (T + G - 1 + TC - 1) / TC;  // enough for the most skewed row

    static_assert(!MERGE || (LPP == 1 && R <= kWave), "line merging is written for one line per piece");
    static_assert(!ELEM || (MERGE && (R * 4) % 128 == 0), "rows that are not whole vectors need merged lines and line-aligned tiles");
    LoihiState st = {0, 0, 0};
    float4 x[NB];
    float headC[MERGE && kCur ? G : 1], headV[MERGE && kVol ? G : 1];  // results of this row's first line (MERGE)
    uint32_t headFired = 0;
    uint32_t prevFired = 0;  // undelayed spike bits of this row's previous group

    auto rows_of = [&](int64_t t) { return static_cast<int>(min(static_cast<int64_t>(R), rows - t * R)); };
    // samples by which row r of tile t starts after a 128-byte boundary
    auto skew_base = [&](int64_t t) {
        return static_cast<int>((reinterpret_cast<uintptr_t>(w + t * R * static_cast<int64_t>(T)) >> 2) & 31);
    };
    auto issue = [&](int64_t t, int j) {
        const BufferRsrc bufW = make_buffer(w + t * R * static_cast<int64_t>(T));
        const int nRows = rows_of(t);
        const int o0 = skew_base(t);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            const int r = b * RPI + subRow;
            const int time = TC * j - ((o0 + r * T) & 31) + col;
            // any sample of the vector inside the row (with whole-vector rows: all or none)
            x[b] = buffer_load4<kCached>(bufW, masked_offset(r < nRows && time + 3 >= 0 && time < T, (r * T + time) * 4), 0);
        }
    };

    int64_t t = blockIdx.x;
    int j = 0;
    if (t >= tiles) return;
    issue(t, j);
    {
        // The loop below keeps one piece of loads and one piece of stores in flight and waits only
        // for the loads ("all but the most recent memory instructions", 3*NB of them with all outputs).  Entering it with the
        // same number of stores behind the first loads - dropped by the range check - lets the
        // compiler use that count on every trip instead of waiting for everything.
        const BufferRsrc none = make_buffer(w);
#pragma unroll
        for (int b = 0; b < (OUTS == 0 ? 3 : OUTS) * NB; ++b)  // distinct (all out-of-range) addresses, so none is folded away
            buffer_store4(none, kOutOfRange + 16 * b, 0, make_float4(static_cast<float>(b), 0.0f, 0.0f, 0.0f));
    }
    while (t < tiles) {
        const int nRows = rows_of(t);
        const int o0 = skew_base(t);
        const bool last = j + 1 == pieces;

#pragma unroll
        for (int b = 0; b < NB; ++b) *reinterpret_cast<float4 *>(tileC + (b * RPI + subRow) * P + col) = x[b];
        wave_sync();
        {
            const int64_t tn = last ? t + gridDim.x : t;
            if (tn < tiles) issue(tn, last ? 0 : j + 1);
        }

        // ---- sequential update: lane = row; this lane's column c is its sample TC*j - o + c
        if (R == kWave || lane < R) {
            if (j == 0) { st = {0, 0, 0}; prevFired = 0; }
            float *mineC = tileC + lane * P;
            float *mineV = tileV + (kVol ? lane * P : 0);
            const int tRow = TC * j - ((o0 + lane * T) & 31);
            // pieces that lie inside every row need no per-sample checks
            const bool inside = j >= 1 && TC * (j + 1) <= T;
#pragma unroll
            for (int g = 0; g < LPP; ++g) {
                const int c0 = g * G;
                float in[G], cur[G], vol[G];
#pragma unroll
                for (int k = 0; k < G; k += 4) {
                    const float4 q = *reinterpret_cast<const float4 *>(mineC + c0 + k);
                    in[k] = q.x; in[k + 1] = q.y; in[k + 2] = q.z; in[k + 3] = q.w;
                }
                uint32_t fired = 0;
                bool small = inside && p.keepI <= 4096u && p.keepV <= 4096u;
                if (small) {
                    // on the assumption that both states stay small; checked afterwards
                    const LoihiState before = st;
                    int lo = min(st.current, st.voltage), hi = max(st.current, st.voltage);
#pragma unroll
                    for (int k = 0; k < G; ++k) fired |= loihi_step_small(st, p, in[k], cur[k], vol[k], lo, hi) << k;
                    small = __builtin_amdgcn_ballot_w64(lo <= -kLoihiSmall || hi >= kLoihiSmall) == 0;
                    if (!small) { st = before; fired = 0; }
                }
                if (small) {
                } else if (inside) {
#pragma unroll
                    for (int k = 0; k < G; ++k) fired |= loihi_step(st, p, in[k], cur[k], vol[k]) << k;
                } else {
#pragma unroll
                    for (int k = 0; k < G; ++k) {
                        // sample 0 is forced to zero and leaves the state untouched; samples outside
                        // the row do not exist
                        const int time = tRow + c0 + k;
                        const bool ok = time >= 1 && time < T;
                        LoihiState next = st;
                        float c, vo;
                        const uint32_t spike = loihi_step(next, p, in[k], c, vo);
                        st.current = ok ? next.current : st.current;
                        st.voltage = ok ? next.voltage : st.voltage;
                        st.countdown = ok ? next.countdown : st.countdown;
                        cur[k] = ok ? c : 0.0f;
                        vol[k] = ok ? vo : 0.0f;
                        fired |= (ok ? spike : 0u) << k;
                    }
                }
#pragma unroll
                for (int k = 0; k < G; k += 4) {
                    if (kCur) *reinterpret_cast<float4 *>(mineC + c0 + k) = make_float4(cur[k], cur[k + 1], cur[k + 2], cur[k + 3]);
                    if (kVol) *reinterpret_cast<float4 *>(mineV + c0 + k) = make_float4(vol[k], vol[k + 1], vol[k + 2], vol[k + 3]);
                }
                // the delayed bits; those that would land beyond the end of the row are dropped
                // (the end of this row's last line belongs to the next row)
                uint32_t out = loihi_delayed(fired, prevFired, p.delay);
                prevFired = fired;
                if (!inside) {
                    const int left = T - (tRow + c0);  // samples of the row from this group on
                    out &= left >= G ? 0xffffffffu : (left > 0 ? (1u << left) - 1u : 0u);
                }
                masks[lane * LPP + g] = out;
                if (MERGE && j == 0) {
#pragma unroll
                    for (int k = 0; k < G; ++k) {
                        if (kCur) headC[k] = cur[k];
                        if (kVol) headV[k] = vol[k];
                    }
                    headFired = out;
                }
            }
            if (MERGE && j > 0) {
                // hand this row's first line over to the row above when that row reaches it
                const int skew = (o0 + lane * T) & 31;             // samples of that line owned by the row above
                const int skewAbove = (o0 + (lane - 1) * T) & 31;
                const int lastAbove = (T - 1 + skewAbove) >> 5;    // piece in which the row above ends
                if (lane > 0 && lane < nRows && skew > 0 && j == lastAbove) {
                    float *aboveC = tileC + (lane - 1) * P;
                    float *aboveV = tileV + (kVol ? (lane - 1) * P : 0);
                    if (ELEM) {
#pragma unroll
                        for (int k = 0; k < G; ++k) {
                            if (k >= skew) {
                                if (kCur) aboveC[k] = headC[k];
                                if (kVol) aboveV[k] = headV[k];
                            }
                        }
                    } else {
#pragma unroll
                        for (int k = 0; k < G; k += 4) {
                            if (k >= skew) {
                                if (kCur) *reinterpret_cast<float4 *>(aboveC + k) = make_float4(headC[k], headC[k + 1], headC[k + 2], headC[k + 3]);
                                if (kVol) *reinterpret_cast<float4 *>(aboveV + k) = make_float4(headV[k], headV[k + 1], headV[k + 2], headV[k + 3]);
                            }
                        }
                    }
                    masks[lane - 1] |= headFired;
                }
            }
        }
        wave_sync();

        // ---- retire: whole lines of current, voltage and spikes
        {
            const int64_t base = t * R * static_cast<int64_t>(T);
            const BufferRsrc bufS = make_buffer(s + base);
            const BufferRsrc bufV = make_buffer((v ? v : s) + base);
            const BufferRsrc bufU = make_buffer((u ? u : s) + base);
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                const int r = b * RPI + subRow;
                const int skew = (o0 + r * T) & 31;
                const int time = TC * j - skew + col;
                bool ok = r < nRows && time >= 0 && time < T;
                if (MERGE) {
                    // a row's first line, when shared, goes out with the last line of the row above ..
                    if (j == 0 && r > 0 && skew > 0) ok = false;
                    // .. whose last line therefore extends into the row below
                    if (r + 1 < nRows && time >= T && j == ((T - 1 + skew) >> 5)) ok = true;
                }
                const int off = masked_offset(ok, (r * T + time) * 4);
                const uint32_t m = masks[r * LPP + (col >> 5)] >> (col & 31);
                // (OUTS = 0: an output that is not wanted is masked, not skipped - with a fixed number of stores per trip
                // the wait for the next piece's loads can leave all of them in flight, not just the spikes')
                if (OUTS == 0) buffer_store4(bufU, u ? off : kOutOfRange, 0, *reinterpret_cast<const float4 *>(tileC + r * P + col));
                if (OUTS == 2 || OUTS == 0)
                    buffer_store4(bufV, (OUTS == 2 || v) ? off : kOutOfRange, 0, *reinterpret_cast<const float4 *>(tileV + (kVol ? r * P + col : 0)));
                buffer_store4(bufS, off, 0,
                              make_float4((m & 1u) ? 1.0f : 0.0f, (m & 2u) ? 1.0f : 0.0f,
                                          (m & 4u) ? 1.0f : 0.0f, (m & 8u) ? 1.0f : 0.0f));
            }
        }
        wave_sync();

        if (last) { t += gridDim.x; j = 0; }
        else ++j;
    }
}

}  // namespace slayer

namespace slayer {

static int launch_loihi(float *s, float *v, float *u, const float *w, int64_t nNeurons, int64_t T,
                        uint32_t wgtExp, int32_t theta, uint32_t iDecay, uint32_t vDecay, uint32_t refDelay,
                        int delaySteps, hipStream_t st)
{
    if (nNeurons < 0 || T < 0) return SLAYER_EINVAL;
    if (refDelay == 0 || wgtExp > 25 || refDelay > 0x7fffffffu) return SLAYER_EINVAL;
    if (delaySteps < 0) return SLAYER_EINVAL;
    if (delaySteps > 31) return SLAYER_EUNSUPPORTED;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!s || !w) return SLAYER_EINVAL;

    LoihiParams p;
    p.weightShift = 6 + wgtExp;  // weight scale 1 << (6 + wgtExp)
    p.keepI = 4096u - iDecay;
    p.keepV = 4096u - vDecay;
    p.refDelay = static_cast<int>(refDelay);
    p.vDecay = vDecay;
    p.theta = theta;
    p.delay = delaySteps;

    if (!generic_forced() && T <= kBufferMaxT) {
        constexpr int kRows = 32, kPiece = LOIHI_PIECE;
        const int64_t tiles = ceil_div(nNeurons, kRows);
        // rows shorter than a piece travel whole; the update goes in groups of 32 columns
        const int Tc = T < kPiece ? static_cast<int>(T) : kPiece;
        const int cols = (Tc + 31) & ~31;
        const int P = cols + 4;  // 4 (mod 32): rows are 16-byte aligned and start in different banks
        const int MP = cols / 32 + 1;
        const size_t lds = (static_cast<size_t>(2 * kRows) * P + kRows * MP) * sizeof(float);
        const int64_t resident = static_cast<int64_t>(compute_units()) * (160 * 1024 / static_cast<int64_t>(lds));
        const unsigned grid = static_cast<unsigned>(tiles < resident ? tiles : resident);
        // outputs the caller does not want (null) constrain nothing
        const bool vec = (T % 4 == 0) && aligned16(s) && aligned16(v) && aligned16(u) && aligned16(w);
        const uintptr_t phase = reinterpret_cast<uintptr_t>(w) & 127;
        const bool samePhase = (reinterpret_cast<uintptr_t>(s) & 127) == phase &&
                               (!v || (reinterpret_cast<uintptr_t>(v) & 127) == phase) &&
                               (!u || (reinterpret_cast<uintptr_t>(u) & 127) == phase);
        const bool elem = (T % 4 != 0) && T >= 64 && (nNeurons * T) % 4 == 0 && aligned16(s) && aligned16(v) &&
                          aligned16(u) && aligned16(w) && samePhase && LOIHI_LPP == 1 && LOIHI_ROWS == 32;
        // Without the current among the outputs the sequential update, not the stores, sets the pace:
        // 64 rows per wavefront then use every lane in it (measured on (8,16,32,32,300): spikes alone
        // 80 us against 112 us, spikes and voltage 112 us against 120 us; all three outputs 145-249 us
        // against 147-237 us, so those keep 32 rows).
        const bool wide = !u && LOIHI_ROWS == 32;
        auto lines_grid = [&](int rowsPerTile, int lpp, int tilesInLds, int64_t &lineTiles) {
            lineTiles = ceil_div(nNeurons, rowsPerTile);
            const int64_t ldsBytes = (static_cast<int64_t>(tilesInLds) * rowsPerTile * (32 * lpp + 4) + rowsPerTile * lpp) * 4 + 16;
            const int64_t fit = static_cast<int64_t>(compute_units()) * (160 * 1024 / ldsBytes);
            return dim3(static_cast<unsigned>(lineTiles < fit ? lineTiles : fit));
        };
#define SLAYER_LOIHI_LINES(R_, LPP_, MERGE_, ELEM_, OUTS_)                                                           \
    do {                                                                                                             \
        int64_t lineTiles;                                                                                           \
        const dim3 grid = lines_grid(R_, LPP_, (OUTS_) == 1 ? 1 : 2, lineTiles);                                     \
        hipLaunchKernelGGL((loihi_lines_kernel<R_, LPP_, MERGE_, ELEM_, OUTS_>), grid, dim3(kWave), 0, st, s, v, u, \
                           w, nNeurons, static_cast<int>(T), lineTiles, p);                                          \
    } while (0)
        if (elem) {
            if (wide && !v) SLAYER_LOIHI_LINES(64, 1, true, true, 1);
            else if (wide) SLAYER_LOIHI_LINES(64, 1, true, true, 2);
            else SLAYER_LOIHI_LINES(32, 1, true, true, 0);
            return launch_status();
        }
        if (vec && samePhase) {
            constexpr int kR = LOIHI_ROWS, kLpp = LOIHI_LPP;
            if (kLpp == 1 && T >= 64 && wide && !v) SLAYER_LOIHI_LINES(64, 1, true, false, 1);
            else if (kLpp == 1 && T >= 64 && wide) SLAYER_LOIHI_LINES(64, 1, true, false, 2);
            else if (kLpp == 1 && T >= 64) SLAYER_LOIHI_LINES(kR, kLpp, kLpp == 1, false, 0);
            else SLAYER_LOIHI_LINES(kR, kLpp, false, false, 0);
            return launch_status();
        }
#undef SLAYER_LOIHI_LINES
        if (vec)
            hipLaunchKernelGGL((loihi_tile_kernel<true, kRows, kPiece>), dim3(grid), dim3(kWave), lds, st, s, v, u,
                               w, nNeurons, static_cast<int>(T), Tc, P, MP, tiles, p);
        else
            hipLaunchKernelGGL((loihi_tile_kernel<false, kRows, kPiece>), dim3(grid), dim3(kWave), lds, st, s, v,
                               u, w, nNeurons, static_cast<int>(T), Tc, P, MP, tiles, p);
        return launch_status();
    }
    const int64_t blocks = ceil_div(nNeurons, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    hipLaunchKernelGGL(loihi_generic_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, st, s, v,
                       u, w, nNeurons, T, p);
    return launch_status();
}

}  // namespace slayer

extern "C" int slayer_loihi_get_spikes_f32(float *s, float *v, float *u, const float *w,
                                           int64_t nNeurons, int64_t T, uint32_t wgtExp, int32_t theta,
                                           uint32_t iDecay, uint32_t vDecay, uint32_t refDelay,
                                           void *stream)
{
    if (nNeurons > 0 && T > 0 && (!v || !u)) return SLAYER_EINVAL;
    return slayer::launch_loihi(s, v, u, w, nNeurons, T, wgtExp, theta, iDecay, vDecay, refDelay, 0,
                                static_cast<hipStream_t>(stream));
}

extern "C" int slayer_loihi_get_spikes_delayed_f32(float *s, float *v, float *u, const float *w,
                                                   int64_t nNeurons, int64_t T, uint32_t wgtExp, int32_t theta,
                                                   uint32_t iDecay, uint32_t vDecay, uint32_t refDelay,
                                                   int32_t delaySteps, void *stream)
{
    return slayer::launch_loihi(s, v, u, w, nNeurons, T, wgtExp, theta, iDecay, vDecay, refDelay, delaySteps,
                                static_cast<hipStream_t>(stream));
}

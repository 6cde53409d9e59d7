// PSP filtering with the alpha kernel that SLAYER's layers use, h[k] = mult * (k Ts / tau) * exp(1 - k Ts / tau)
// for k < L (src/slayer.py:98-123), as a recursion instead of an L-tap sum:
//
//   conv: y[t] = Ts * sum_{k<L} h[k] x[t-k]          corr: y[t] = Ts * sum_{k<L} h[k] x[t+k]
//
// With a = exp(-Ts / tau) and g = mult * e * Ts / tau the kernel is h[k] = g k a^k.  The two running sums
//
//   p[t] = sum_{k>=0} a^k x[t-k]   = a p[t-1] + x[t]
//   q[t] = sum_{k>=0} k a^k x[t-k] = a (q[t-1] + p[t-1])
//
// give the untruncated response g q[t]; the taps from L on amount to a^L (L p[t-L] + q[t-L]) = a^L r[t-L] with
// r = L p + q, so
//
//   y[t] = Ts g (q[t] - a^L r[t-L]).
//
// About 10 floating-point operations per sample instead of 2 L: at 77 taps the L-tap sum sits on the FP32 ridge
// of the machine (matrix-pipe bound at 0.47 of HBM peak); the recursion is a memory stream.
//
// A wavefront owns 4 consecutive rows - always a run of whole 16-byte vectors - in LDS as they lie in memory.  Sixteen lanes serve
// a row, each a contiguous segment of its time axis: pass 1 runs the recursion over the segment from zero state,
// a scan over the row's lanes composes the segments (state after n more samples: p' = a^n p,
// q' = a^n (q + n p), plus the run's own sums) into the state in front of each, pass 2 runs the recursion again from the true state and
// leaves q[t] (over x[t]) and r[t] in LDS; then all lanes combine q[t] and r[t -+ L] vector by vector on the way
// out.  The correlation is the same on the reversed time axis.  Every output is a sum of the same products as
// the L-tap chain (with a^k taken as a product of a's instead of one rounded tap), added in another order, and
// the difference of the two running sums: it agrees with the chain to rounding relative to the sum of the
// magnitudes of the UNTRUNCATED response's terms, sum_k |x[t-k]| g k a^k - a bound that also holds where the
// truncated sum is small or zero (behind a large sample that has left the window).  A tile that holds a
// non-finite sample is filtered with the L-tap chain from the given filter, so that infinities and NaNs reach
// exactly the samples the reference lets them reach.
#include "common.h"
#include <type_traits>

namespace slayer {

// Rows per wavefront.  4 rows of T = 300 are 4800 bytes, whole 64-byte blocks; their two copies in LDS take 9.6 KB, so
// 16 wavefronts fit a compute unit (8 rows per wavefront, 8 wavefronts: 131 us instead of 96 us on the benchmark tensor).
constexpr int kAlphaRows = 4;
constexpr int kAlphaMaxT = 512;   // two copies of 4 rows in LDS: 16 KiB at most

struct AlphaArgs {
    float *out;
    const float *in, *filt;
    int64_t rows;
    int T, L;
    float a;            // exp(-Ts / tau)
    float aSeg[2];      // a^n for segments of perRow / parts and perRow / parts + 1 vectors (n = 4 times that)
    float aL;           // a^L
    float scale;        // Ts * mult * e * Ts / tau
    float Ts;
    // GATE = 1: the samples are in * gain * exp(-|u - theta| / tauRho) (the spike function's surrogate gradient),
    // applied on the way into LDS.  GATE = 2: the same factor, of the same positions, multiplies the results on the
    // way out instead, after `add` (same shape, may be null) has been added to them.
    const float *u;
    float theta, tauRho, gain;
    const float *add;
};

// VEC: rows are whole 16-byte vectors (T % 4 == 0).  Otherwise a tile of 4 rows is still a contiguous, 16-byte aligned
// run of whole vectors (4 T floats) and travels the same way, but a vector may hold the end of one row and the start of
// the next: the passes then read and write LDS sample by sample, and the way out places every sample in its row.
template <bool CAUSAL, int R, int GATE, bool VEC>
__global__ __launch_bounds__(64) void alpha_psp_kernel(AlphaArgs p)
{
    constexpr bool GATED = GATE == 1, GATED_OUT = GATE == 2;
    constexpr int kParts = kWave / R;
    constexpr int NB = (R * (kAlphaMaxT / 4) + kWave - 1) / kWave;  // vectors per lane of a tile, at most
    extern __shared__ __align__(16) float lds[];
    const int T = p.T, P = p.T, L = p.L;   // rows follow each other in LDS as in memory
    float *Q = lds;            // [R][T]: x, then q
    float *Rr = lds + R * P;   // [R][T]: r

    const int lane = threadIdx.x;
    const int perRow = T >> 2;                 // (VEC: vectors per row)
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), p.rows - row0));
    const int nVec = (nRows * T) >> 2;         // the tile is whole vectors: the host checked (rows * T) % 4 == 0
    const int tileVec = (R * T) >> 2;

    // ---- the tile, one contiguous run of vectors, in LDS exactly as it lies in memory (rows behind the last one
    //      arrive as zeros): vector e of the tile is vector e of LDS, no index arithmetic
    bool bad = false;
    float4 gu[GATE != 0 ? NB : 1];  // the membrane potentials of this lane's vectors (GATE = 2: kept for the way out)
    {
        const BufferRsrc bufIn = make_buffer(p.in + row0 * static_cast<int64_t>(T), nVec * 16);
        const BufferRsrc bufU = make_buffer((GATE != 0 ? p.u : p.in) + row0 * static_cast<int64_t>(T), nVec * 16);
        float4 x[NB];
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b * kWave < tileVec) {
                x[b] = buffer_load4<kCached>(bufIn, (lane + b * kWave) * 16, 0);
                if (GATE != 0) gu[b] = buffer_load4<kCached>(bufU, (lane + b * kWave) * 16, 0);
            }
        }
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b * kWave < tileVec) {
                if (lane + b * kWave < tileVec) {
                    if (GATED)
                        x[b] = make_float4(x[b].x * spike_pdf(gu[b].x, p.theta, p.tauRho, p.gain),
                                           x[b].y * spike_pdf(gu[b].y, p.theta, p.tauRho, p.gain),
                                           x[b].z * spike_pdf(gu[b].z, p.theta, p.tauRho, p.gain),
                                           x[b].w * spike_pdf(gu[b].w, p.theta, p.tauRho, p.gain));
                    *reinterpret_cast<float4 *>(Q + 4 * (lane + b * kWave)) = x[b];
                    // infinite or NaN (or four samples that add up to more than fp32 holds, which only costs time)
                    bad |= ((x[b].x + x[b].y) + (x[b].z + x[b].w)) * 0.0f != 0.0f;
                }
            }
        }
    }
    const bool chains = __builtin_amdgcn_ballot_w64(bad) != 0;
    wave_sync();

    if (chains) {
        // a non-finite sample: the tile's outputs as the sequential chains over the valid taps, from memory
        for (int e = lane; e < nRows * T; e += kWave) {
            const int r = e / T, t = e - r * T;
            const float *x = p.in + (row0 + r) * static_cast<int64_t>(T);
            const int taps = CAUSAL ? min(t + 1, L) : min(T - t, L);
            const float *gu = GATED ? p.u + (row0 + r) * static_cast<int64_t>(T) : nullptr;
            auto sample = [&](int i) { return GATED ? x[i] * spike_pdf(gu[i], p.theta, p.tauRho, p.gain) : x[i]; };
            float acc = 0.0f;
            for (int k = 0; k < taps; ++k) acc = __builtin_fmaf(sample(CAUSAL ? t - k : t + k), p.filt[k], acc);
            acc *= p.Ts;
            if (GATED_OUT) {
                const int64_t at = (row0 + r) * static_cast<int64_t>(T) + t;
                if (p.add) acc += p.add[at];
                acc *= spike_pdf(p.u[at], p.theta, p.tauRho, p.gain);
            }
            p.out[(row0 + r) * static_cast<int64_t>(T) + t] = acc;
        }
        return;
    }

    // ---- lane (row r, part j): a segment of the row's logical time axis - vectors [v0, v1) (VEC) or samples
    //      [v0, v1) - where logical time runs forward for the convolution and backward for the correlation (logical
    //      vector V = memory vector perRow - 1 - V, mirrored; logical sample i = memory sample T - 1 - i)
    const int r = lane / kParts, j = lane - r * kParts;
    const int units = VEC ? perRow : T;
    const int v0 = (j * units) / kParts, v1 = ((j + 1) * units) / kParts;
    const float a = p.a;
    float *q4 = Q + r * P, *r4 = Rr + r * P;
    auto vector_at = [&](int V) { return (CAUSAL ? V : perRow - 1 - V) << 2; };
    auto sample_at = [&](int i) { return CAUSAL ? i : T - 1 - i; };
    auto step = [&](float &pp, float &qq, float x) {
        qq = a * (qq + pp);                 // q[t] = a (q[t-1] + p[t-1])
        pp = __builtin_fmaf(a, pp, x);      // p[t] = a p[t-1] + x[t]
    };
    float sp = 0.0f, sq = 0.0f;   // the segment's own sums (its end state from a zero start)
    if constexpr (VEC) {
#pragma unroll 2
        for (int V = v0; V < v1; ++V) {
            const float4 x = *reinterpret_cast<const float4 *>(q4 + vector_at(V));
            step(sp, sq, CAUSAL ? x.x : x.w);
            step(sp, sq, CAUSAL ? x.y : x.z);
            step(sp, sq, CAUSAL ? x.z : x.y);
            step(sp, sq, CAUSAL ? x.w : x.x);
        }
    } else {
#pragma unroll 4
        for (int i = v0; i < v1; ++i) step(sp, sq, q4[sample_at(i)]);
    }
    // The state in front of every segment.  A run of n samples takes a state (p, q) to (a^n p, a^n (q + n p)) plus
    // its own sums; runs compose, so an inclusive scan over the row's lanes (4 steps of lane-shifting moves, each
    // lane taking in the run that ends d lanes below it) leaves the state behind every segment, and the lane
    // below hands it up.  Lanes without a lane d below take in the empty run (1, 0, 0, 0).
    float cp, cq;
    {
        float rA = p.aSeg[(v1 - v0) - units / kParts], rN = static_cast<float>(VEC ? (v1 - v0) << 2 : v1 - v0), rP = sp, rQ = sq;
        auto below = [&](float own, float identity, auto ctrlTag) {   // row_shr:d as a compile-time constant
            return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity),
                                                                         __builtin_bit_cast(int, own), decltype(ctrlTag)::value,
                                                                         0xf, 0xf, false));
        };
        auto take_in = [&](auto ctrlTag) {
            const float lA = below(rA, 1.0f, ctrlTag), lN = below(rN, 0.0f, ctrlTag), lP = below(rP, 0.0f, ctrlTag),
                        lQ = below(rQ, 0.0f, ctrlTag);
            rQ = __builtin_fmaf(rA, __builtin_fmaf(rN, lP, lQ), rQ);
            rP = __builtin_fmaf(rA, lP, rP);
            rA *= lA;
            rN += lN;
        };
        static_assert(kParts == 16, "a row's lanes are one row of the lane-shifting moves");
        take_in(std::integral_constant<int, 0x111>{});
        take_in(std::integral_constant<int, 0x112>{});
        take_in(std::integral_constant<int, 0x114>{});
        take_in(std::integral_constant<int, 0x118>{});
        cp = below(rP, 0.0f, std::integral_constant<int, 0x111>{});
        cq = below(rQ, 0.0f, std::integral_constant<int, 0x111>{});
    }
    // pass 2: q over x, r next to it
    {
        const float fL = static_cast<float>(L);
        float pp = cp, qq = cq;
        if constexpr (VEC) {
#pragma unroll 2
            for (int V = v0; V < v1; ++V) {
                const int at = vector_at(V);
                const float4 x = *reinterpret_cast<const float4 *>(q4 + at);
                float qv[4], rv[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float xe = CAUSAL ? (e == 0 ? x.x : e == 1 ? x.y : e == 2 ? x.z : x.w)
                                            : (e == 0 ? x.w : e == 1 ? x.z : e == 2 ? x.y : x.x);
                    step(pp, qq, xe);
                    qv[e] = qq;
                    rv[e] = __builtin_fmaf(fL, pp, qq);
                }
                *reinterpret_cast<float4 *>(q4 + at) = CAUSAL ? make_float4(qv[0], qv[1], qv[2], qv[3]) : make_float4(qv[3], qv[2], qv[1], qv[0]);
                *reinterpret_cast<float4 *>(r4 + at) = CAUSAL ? make_float4(rv[0], rv[1], rv[2], rv[3]) : make_float4(rv[3], rv[2], rv[1], rv[0]);
            }
        } else {
#pragma unroll 4
            for (int i = v0; i < v1; ++i) {
                const int at = sample_at(i);
                step(pp, qq, q4[at]);
                q4[at] = qq;
                r4[at] = __builtin_fmaf(fL, pp, qq);
            }
        }
    }
    wave_sync();

    // ---- out: y[t] = scale (q[t] - a^L r[t -+ L]); the four r of a vector lie in two aligned vectors, L & 3
    //      samples off (the same for every lane)
    {
        const BufferRsrc bufOut = make_buffer(p.out + row0 * static_cast<int64_t>(T), nVec * 16);
        const float aL = p.aL, scale = p.scale;
        const int shift = CAUSAL ? -L : L;           // r[t + shift]
        const int lo = shift >> 2, off = shift & 3;  // r[4 c + e + shift] = element (e + off) of vectors c + lo, c + lo + 1
        static_assert(R == 4, "the row of a vector or sample from three comparisons");
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            if (b * kWave < tileVec) {
                const int e = min(lane + b * kWave, tileVec - 1);  // (lanes behind the tile: their stores are dropped)
                const float4 qv = *reinterpret_cast<const float4 *>(Q + 4 * e);
                float4 rs;
                if constexpr (VEC) {
                    const int row = (e >= perRow ? 1 : 0) + (e >= 2 * perRow ? 1 : 0) + (e >= 3 * perRow ? 1 : 0);
                    const int c = e - row * perRow;
                    const int ca = c + lo, cb = ca + 1;
                    const float4 zero = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                    const float4 ra = (ca >= 0 && ca < perRow) ? *reinterpret_cast<const float4 *>(Rr + 4 * (e + lo)) : zero;
                    const float4 rb = (off != 0 && cb >= 0 && cb < perRow) ? *reinterpret_cast<const float4 *>(Rr + 4 * (e + lo + 1)) : zero;
                    if (off == 0) rs = ra;
                    else if (off == 1) rs = make_float4(ra.y, ra.z, ra.w, rb.x);
                    else if (off == 2) rs = make_float4(ra.z, ra.w, rb.x, rb.y);
                    else rs = make_float4(ra.w, rb.x, rb.y, rb.z);
                } else {
                    float rk[4];
#pragma unroll
                    for (int k = 0; k < 4; ++k) {   // sample g of the tile lies in row g / T; its partner r must lie in the same row
                        const int g = 4 * e + k;
                        const int row = (g >= T ? 1 : 0) + (g >= 2 * T ? 1 : 0) + (g >= 3 * T ? 1 : 0);
                        const int t = g - row * T + shift;
                        rk[k] = (t >= 0 && t < T) ? Rr[g + shift] : 0.0f;
                    }
                    rs = make_float4(rk[0], rk[1], rk[2], rk[3]);
                }
                float4 y = make_float4(scale * __builtin_fmaf(-aL, rs.x, qv.x), scale * __builtin_fmaf(-aL, rs.y, qv.y),
                                       scale * __builtin_fmaf(-aL, rs.z, qv.z), scale * __builtin_fmaf(-aL, rs.w, qv.w));
                if (GATED_OUT) {
                    if (p.add) {
                        const BufferRsrc bufAdd = make_buffer(p.add + row0 * static_cast<int64_t>(T), nVec * 16);
                        const float4 more = buffer_load4<kCached>(bufAdd, (lane + b * kWave) * 16, 0);
                        y = make_float4(y.x + more.x, y.y + more.y, y.z + more.z, y.w + more.w);
                    }
                    y = make_float4(y.x * spike_pdf(gu[b].x, p.theta, p.tauRho, p.gain), y.y * spike_pdf(gu[b].y, p.theta, p.tauRho, p.gain),
                                    y.z * spike_pdf(gu[b].z, p.theta, p.tauRho, p.gain), y.w * spike_pdf(gu[b].w, p.theta, p.tauRho, p.gain));
                }
                buffer_store4(bufOut, (lane + b * kWave) * 16, 0, y);
            }
        }
    }
}

// ---- rows longer than kAlphaMaxT: the same recursion piece by piece ---------------------------------------------
// A wavefront owns 4 rows and walks them in pieces of kPieceT samples along the logical time axis (forward for the
// convolution, backward for the correlation).  What a piece needs from the ones before it is three numbers per row -
// the running sums p and q at its start, composed into the lanes' scan like one more segment - and the last H >= L
// values of r, kept in front of the piece's own r in LDS, so that r[t - L] is read the same way everywhere (zeros in
// front of the row).  LDS holds a piece in logical order: for the correlation the vectors and their elements are
// mirrored between memory and LDS, which costs nothing (a lane loads and stores the same memory vector either way)
// and leaves one form of the passes.  The loads of the next piece are issued before the passes over this one.
constexpr int kPieceT = 256;              // samples per row and piece: 64 vectors, one per lane on the way in and out
constexpr int kPieceMaxL = kPieceT;       // r[t - L] lies in this piece or the one before

struct AlphaPieces {
    int H;              // history samples of r per row: L rounded up to whole vectors
    float aPow[5];      // a^16, a^32, a^64, a^128, a^256: runs of 1, 2, 4, 8 and 16 of a full piece's segments
    float aSegLast[2];  // a^n for the last piece's segments of units / 16 and units / 16 + 1 vectors
};

// OFF = H - L (0 .. 3): how far r[t - L] lies from a vector boundary - a template parameter, so that the way out is
// straight-line code: together with loads and stores that are masked instead of branched around, every trip of the
// piece loop issues the same memory instructions, and the wait for a piece's loads can leave the younger stores of the
// piece before it in flight.
template <bool CAUSAL, int GATE, int OFF>
__global__ __launch_bounds__(64) void alpha_psp_pieces_kernel(AlphaArgs p, AlphaPieces pc)
{
    constexpr bool GATED = GATE == 1, GATED_OUT = GATE == 2;
    constexpr int R = kAlphaRows, kParts = kWave / R, PT = kPieceT, PV = PT / 4, SEG = PV / kParts;
    static_assert(R == 4 && PV == kWave && SEG == 4, "lane c moves vector c of every row's piece; segments of 4 vectors");
    extern __shared__ __align__(16) float lds[];
    const int T = p.T, L = p.L, H = pc.H, HV = H >> 2;
    const int pitch = H + PT;
    float *Q = lds;             // [R][PT]: x, then q, logical order
    float *Rr = lds + R * PT;   // [R][H + PT]: the last H values of r of the piece before, then this piece's

    const int lane = threadIdx.x;
    const int perRow = T >> 2;
    const int nFull = perRow / PV, lastUnits = perRow - nFull * PV;   // full pieces, vectors per row of a shorter last one
    const int64_t row0 = static_cast<int64_t>(blockIdx.x) * R;
    const int nRows = static_cast<int>(min(static_cast<int64_t>(R), p.rows - row0));
    const int rowBytes = T * 4;
    const int tileBytes = nRows * rowBytes;   // rows behind the last one read zeros, their stores are dropped
    const BufferRsrc bufIn = make_buffer(p.in + row0 * static_cast<int64_t>(T), tileBytes);
    const BufferRsrc bufU = make_buffer((GATE != 0 ? p.u : p.in) + row0 * static_cast<int64_t>(T), tileBytes);
    const BufferRsrc bufAdd = make_buffer((GATED_OUT && p.add ? p.add : p.in) + row0 * static_cast<int64_t>(T), tileBytes);
    const BufferRsrc bufOut = make_buffer(p.out + row0 * static_cast<int64_t>(T), tileBytes);
    const bool hasAdd = GATED_OUT && p.add != nullptr;

    // byte offset of this lane's vector of piece k inside a row (the same on the way in and on the way out; behind the
    // row's end: out of range, which reads zeros and drops stores)
    auto lane_offset = [&](int k) {
        const int V = k * PV + lane;
        return masked_offset(V < perRow, (CAUSAL ? V : perRow - 1 - V) * 16);
    };
    auto mirrored = [](float4 v) { return CAUSAL ? v : make_float4(v.w, v.z, v.y, v.x); };
    // Where vector V of a row's piece lies in LDS.  The lanes of a row walk segments of 4 vectors: laid out as they
    // come, the vectors that 8 lanes read together would fall into two of the 8 groups of banks.  Exchanging the low
    // bits of the position with the segment's number spreads them over all 8, for the lanes that walk segments and for
    // the lanes that move consecutive vectors alike.
    auto swz = [](int V) { return V ^ ((V >> 3) & 7); };
    auto r_at = [&](int w) { return 4 * (w < HV ? w : HV + swz(w - HV)); };   // vector w of a row's r, history included

    for (int b = 0; b < R; ++b)
        for (int c = lane; c < HV; c += kWave)
            *reinterpret_cast<float4 *>(Rr + b * pitch + 4 * c) = make_float4(0.0f, 0.0f, 0.0f, 0.0f);

    // Two sets of registers take turns: a piece's loads are issued two pieces ahead, behind the stores of the piece that
    // has just left the set, so a piece and a half of loads is in flight while a piece is worked on.
    constexpr int NG = GATE != 0 ? R : 1, NM = GATED_OUT ? R : 1;
    float4 xA[R], guA[NG], moreA[NM], xB[R], guB[NG], moreB[NM];
    auto load_piece = [&](int k, float4 (&x)[R], float4 (&gu)[NG], float4 (&more)[NM]) {
        const int at = lane_offset(k);      // (behind the last piece: out of range, zeros that nobody uses)
#pragma unroll
        for (int b = 0; b < R; ++b) {
            x[b] = buffer_load4<kCached>(bufIn, at, b * rowBytes);
            if (GATE != 0) gu[b] = buffer_load4<kCached>(bufU, at, b * rowBytes);
            if (GATED_OUT) more[b] = buffer_load4<kCached>(bufAdd, hasAdd ? at : kOutOfRange, b * rowBytes);
        }
    };
    load_piece(0, xA, guA, moreA);
    // (stores that the range check drops: the first trip then finds the same instructions in flight as the later ones -
    // a piece's loads, the stores of the piece before, the next piece's loads - which is what lets the compiler count them)
#pragma unroll
    for (int b = 0; b < R; ++b) buffer_store4(bufOut, kOutOfRange, b * rowBytes, make_float4(0.0f, 0.0f, 0.0f, 0.0f));
    load_piece(1, xB, guB, moreB);
    const int r = lane / kParts, j = lane - r * kParts;
    const float a = p.a, fL = static_cast<float>(L);
    float carryP = 0.0f, carryQ = 0.0f;   // the row's running sums in front of the piece (the same in all its lanes)
    auto step = [&](float &pp, float &qq, float xe) {
        qq = a * (qq + pp);
        pp = __builtin_fmaf(a, pp, xe);
    };
    auto below = [&](float own, float identity, auto ctrlTag) {   // row_shr:d as a compile-time constant
        return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, identity), __builtin_bit_cast(int, own),
                                                                     decltype(ctrlTag)::value, 0xf, 0xf, false));
    };
    using Shr1 = std::integral_constant<int, 0x111>;
    using Shr2 = std::integral_constant<int, 0x112>;
    using Shr4 = std::integral_constant<int, 0x114>;
    using Shr8 = std::integral_constant<int, 0x118>;
    static_assert(kParts == 16, "a row's lanes are one row of the lane-shifting moves");
    // what stays the same from one full piece to the next: where this lane's vectors lie in LDS (on the way in and out:
    // vector `lane` of every row; in the passes: vectors 4 j .. 4 j + 3 of row r) and the decay over the 16 j samples
    // between the piece's start and this lane's segment
    const int mine = 4 * swz(lane), rMine = r_at(lane), rNext = r_at(lane + 1);
    int seg[SEG];
#pragma unroll
    for (int i = 0; i < SEG; ++i) seg[i] = 4 * swz(SEG * j + i);
    const float frontA = ((j & 1) ? pc.aPow[0] : 1.0f) * ((j & 2) ? pc.aPow[1] : 1.0f) * ((j & 4) ? pc.aPow[2] : 1.0f) *
                         ((j & 8) ? pc.aPow[3] : 1.0f);
    const float frontN = static_cast<float>(4 * SEG * j);

    // One piece.  FULL: all 64 vectors per row, every lane a segment of 4 - the shape of all pieces but possibly the last.
    constexpr int kNone = 0x7fffffff;
    int firstBad = kNone;
    auto piece = [&](auto fullTag, int k, float4 (&x)[R], float4 (&gu)[NG], float4 (&more)[NM]) {
        constexpr bool FULL = decltype(fullTag)::value;
        const int units = FULL ? PV : lastUnits;
        const int at = lane_offset(k);
        // ---- this piece into LDS
#pragma unroll
        for (int b = 0; b < R; ++b) {
            float4 v = x[b];
            if (GATED)
                v = make_float4(v.x * spike_pdf(gu[b].x, p.theta, p.tauRho, p.gain), v.y * spike_pdf(gu[b].y, p.theta, p.tauRho, p.gain),
                                v.z * spike_pdf(gu[b].z, p.theta, p.tauRho, p.gain), v.w * spike_pdf(gu[b].w, p.theta, p.tauRho, p.gain));
            // (lanes behind a shorter last piece hold zeros, which nobody reads)
            *reinterpret_cast<float4 *>(Q + b * PT + mine) = mirrored(v);
        }
        wave_sync();
        // ---- lane (row r, part j): vectors [v0, v1) of the row's piece; pass 1 from a zero state
        const int v0 = FULL ? SEG * j : (j * units) / kParts, v1 = FULL ? SEG * j + SEG : ((j + 1) * units) / kParts;
        float *q4 = Q + r * PT, *r4 = Rr + r * pitch + H;
        float sp = 0.0f, sq = 0.0f;
        auto pass1 = [&](int at4) {
            const float4 v = *reinterpret_cast<const float4 *>(q4 + at4);
            step(sp, sq, v.x);
            step(sp, sq, v.y);
            step(sp, sq, v.z);
            step(sp, sq, v.w);
        };
        if constexpr (FULL) {
#pragma unroll
            for (int i = 0; i < SEG; ++i) pass1(seg[i]);
        } else {
            for (int V = v0; V < v1; ++V) pass1(4 * swz(V));
        }
        // ---- the state in front of every segment: an inclusive scan over the row's lanes (a run of n samples takes a
        //      state (p, q) to (a^n p, a^n (q + n p)) plus the run's own sums; each lane takes in the run that ends d
        //      lanes below it), the lane below hands its result up, and the state in front of the piece passes through
        //      the samples in between.  In a full piece the run a lane has gathered before the step over d lanes is d
        //      segments long wherever there is something to take in, so a^n and n are the same for the whole wavefront.
        float cp, cq, tA, tN, rP = sp, rQ = sq;
        if constexpr (FULL) {
            auto take_in = [&](auto ctrlTag, float A, float N) {
                const float lP = below(rP, 0.0f, ctrlTag), lQ = below(rQ, 0.0f, ctrlTag);
                rQ = __builtin_fmaf(A, __builtin_fmaf(N, lP, lQ), rQ);
                rP = __builtin_fmaf(A, lP, rP);
            };
            take_in(Shr1{}, pc.aPow[0], 4.0f * SEG);
            take_in(Shr2{}, pc.aPow[1], 8.0f * SEG);
            take_in(Shr4{}, pc.aPow[2], 16.0f * SEG);
            take_in(Shr8{}, pc.aPow[3], 32.0f * SEG);
            cp = __builtin_fmaf(frontA, carryP, below(rP, 0.0f, Shr1{}));
            cq = __builtin_fmaf(frontA, __builtin_fmaf(frontN, carryP, carryQ), below(rQ, 0.0f, Shr1{}));
            tA = pc.aPow[4];
            tN = static_cast<float>(PT);
        } else {
            float rA = (v1 - v0) > units / kParts ? pc.aSegLast[1] : pc.aSegLast[0], rN = static_cast<float>((v1 - v0) << 2);
            auto take_in = [&](auto ctrlTag) {
                const float lA = below(rA, 1.0f, ctrlTag), lN = below(rN, 0.0f, ctrlTag), lP = below(rP, 0.0f, ctrlTag),
                            lQ = below(rQ, 0.0f, ctrlTag);
                rQ = __builtin_fmaf(rA, __builtin_fmaf(rN, lP, lQ), rQ);
                rP = __builtin_fmaf(rA, lP, rP);
                rA *= lA;
                rN += lN;
            };
            take_in(Shr1{});
            take_in(Shr2{});
            take_in(Shr4{});
            take_in(Shr8{});
            const float eA = below(rA, 1.0f, Shr1{}), eN = below(rN, 0.0f, Shr1{});
            cp = __builtin_fmaf(eA, carryP, below(rP, 0.0f, Shr1{}));
            cq = __builtin_fmaf(eA, __builtin_fmaf(eN, carryP, carryQ), below(rQ, 0.0f, Shr1{}));
            tA = __shfl(rA, lane | (kParts - 1));
            tN = __shfl(rN, lane | (kParts - 1));
        }
        {   // the state behind the piece, from the row's last lane
            const float tP = __shfl(rP, lane | (kParts - 1)), tQ = __shfl(rQ, lane | (kParts - 1));
            const float nextQ = __builtin_fmaf(tA, __builtin_fmaf(tN, carryP, carryQ), tQ);
            carryP = __builtin_fmaf(tA, carryP, tP);
            carryQ = nextQ;
        }
        // An infinite or NaN sample (or sums that outgrow fp32) shows in the running sums behind the piece, and stays in
        // them to the end of the row, where the sum over the taps lets it go after L samples: the first such piece is
        // noted, and the tile is redone from there as chains over the taps once the walk is over.  (Leaving the walk
        // here instead costs every tile: with a way out of the loop the compiler no longer counts the stores in flight
        // and waits for all of them at every piece.)
        firstBad = (firstBad == kNone && __builtin_amdgcn_ballot_w64((carryP + carryQ) * 0.0f != 0.0f) != 0) ? k : firstBad;
        // ---- pass 2: q over x, r behind the history
        {
            float pp = cp, qq = cq;
            auto pass2 = [&](int at4) {
                const float4 v = *reinterpret_cast<const float4 *>(q4 + at4);
                float4 qv, rv;
                step(pp, qq, v.x); qv.x = qq; rv.x = __builtin_fmaf(fL, pp, qq);
                step(pp, qq, v.y); qv.y = qq; rv.y = __builtin_fmaf(fL, pp, qq);
                step(pp, qq, v.z); qv.z = qq; rv.z = __builtin_fmaf(fL, pp, qq);
                step(pp, qq, v.w); qv.w = qq; rv.w = __builtin_fmaf(fL, pp, qq);
                *reinterpret_cast<float4 *>(q4 + at4) = qv;
                *reinterpret_cast<float4 *>(r4 + at4) = rv;
            };
            if constexpr (FULL) {
#pragma unroll
                for (int i = 0; i < SEG; ++i) pass2(seg[i]);
            } else {
                for (int V = v0; V < v1; ++V) pass2(4 * swz(V));
            }
        }
        wave_sync();
        // ---- out: y[i] = scale (q[i] - a^L r[i - L]); r[i - L] of a row's local sample i is Rr[row][OFF + i]: the four
        //      of a vector lie in two aligned vectors of the row's r (history included), OFF samples off
        {
            const float aL = p.aL, scale = p.scale;
            const int c = FULL ? lane : min(lane, units - 1);    // (lanes behind the piece: their stores are dropped)
            const int qAt = FULL ? mine : 4 * swz(c), raAt = FULL ? rMine : r_at(c), rbAt = FULL ? rNext : r_at(c + 1);
#pragma unroll
            for (int b = 0; b < R; ++b) {
                const float4 qv = *reinterpret_cast<const float4 *>(Q + b * PT + qAt);
                const float *rrow = Rr + b * pitch;
                const float4 ra = *reinterpret_cast<const float4 *>(rrow + raAt);
                float4 rs = ra;
                if constexpr (OFF != 0) {
                    const float4 rb = *reinterpret_cast<const float4 *>(rrow + rbAt);
                    if constexpr (OFF == 1) rs = make_float4(ra.y, ra.z, ra.w, rb.x);
                    else if constexpr (OFF == 2) rs = make_float4(ra.z, ra.w, rb.x, rb.y);
                    else rs = make_float4(ra.w, rb.x, rb.y, rb.z);
                }
                float4 y = make_float4(scale * __builtin_fmaf(-aL, rs.x, qv.x), scale * __builtin_fmaf(-aL, rs.y, qv.y),
                                       scale * __builtin_fmaf(-aL, rs.z, qv.z), scale * __builtin_fmaf(-aL, rs.w, qv.w));
                y = mirrored(y);
                if (GATED_OUT) {
                    if (hasAdd) y = make_float4(y.x + more[b].x, y.y + more[b].y, y.z + more[b].z, y.w + more[b].w);
                    y = make_float4(y.x * spike_pdf(gu[b].x, p.theta, p.tauRho, p.gain), y.y * spike_pdf(gu[b].y, p.theta, p.tauRho, p.gain),
                                    y.z * spike_pdf(gu[b].z, p.theta, p.tauRho, p.gain), y.w * spike_pdf(gu[b].w, p.theta, p.tauRho, p.gain));
                }
                buffer_store4(bufOut, at, b * rowBytes, y);
            }
        }
        load_piece(k + 2, x, gu, more);
        // ---- the last H values of this piece's r become the history of the next.  They lie behind the history, so
        //      reading and writing need no synchronisation in between - and nothing may sit in a local array across a
        //      wave_sync: its fence sends such an array through scratch memory, and the wait for that stalls on every
        //      load and store in flight.
        if constexpr (FULL) {
            wave_sync();
            if (lane < HV) {
#pragma unroll
                for (int b = 0; b < R; ++b)
                    *reinterpret_cast<float4 *>(Rr + b * pitch + 4 * lane) = *reinterpret_cast<const float4 *>(Rr + b * pitch + r_at(PV + lane));
            }
            wave_sync();
        }
    };

    int k = 0;
    for (; k + 1 < nFull; k += 2) {
        piece(std::true_type{}, k, xA, guA, moreA);
        piece(std::true_type{}, k + 1, xB, guB, moreB);
    }
    if (k < nFull) {
        piece(std::true_type{}, k, xA, guA, moreA);
        if (lastUnits != 0) piece(std::false_type{}, nFull, xB, guB, moreB);
    } else if (lastUnits != 0) {
        piece(std::false_type{}, nFull, xA, guA, moreA);
    }
    if (firstBad != kNone) {
        // from the piece that met the non-finite sample on, from memory - once the stores of the walk have landed, so
        // that what the chains write is what stays
        __builtin_amdgcn_s_waitcnt(0);
        const int done = firstBad * PT, left = T - done;          // logical samples [done, T) remain
        for (int e = lane; e < nRows * left; e += kWave) {
            const int rr = e / left, i = done + (e - rr * left);
            const int t = CAUSAL ? i : T - 1 - i;
            const int64_t base = (row0 + rr) * static_cast<int64_t>(T);
            const float *xr = p.in + base;
            const int taps = CAUSAL ? min(t + 1, L) : min(T - t, L);
            auto sample = [&](int s) { return GATED ? xr[s] * spike_pdf(p.u[base + s], p.theta, p.tauRho, p.gain) : xr[s]; };
            float acc = 0.0f;
            for (int q = 0; q < taps; ++q) acc = __builtin_fmaf(sample(CAUSAL ? t - q : t + q), p.filt[q], acc);
            acc *= p.Ts;
            if (GATED_OUT) {
                if (p.add) acc += p.add[base + t];
                acc *= spike_pdf(p.u[base + t], p.theta, p.tauRho, p.gain);
            }
            p.out[base + t] = acc;
        }
    }
}

}  // namespace slayer

namespace slayer {

// Launches the recursion, or returns false (nothing launched) for shapes it does not serve.
static bool launch_alpha(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T, int64_t F, float tau,
                         float mult, float Ts, bool causal, const float *u, float theta, float tauRho, float gain,
                         hipStream_t st, bool gateOut = false, const float *add = nullptr)
{
    constexpr int R = kAlphaRows, parts = kWave / R;
    const int64_t tiles = ceil_div(nNeurons, R);
    // rows of whole vectors, or at least a tensor of whole vectors (then every tile of 4 rows is one, too)
    const bool vec = T % 4 == 0;
    if (generic_forced() || (!vec && (nNeurons * T) % 4 != 0) || !aligned16(out) || !aligned16(in) ||
        (u && !aligned16(u)) || (add && !aligned16(add)) || tiles >= (1LL << 31) || F >= (1 << 20))
        return false;
    // longer rows go piece by piece: rows of whole vectors, a kernel no longer than a piece
    const bool pieces = T > kAlphaMaxT;
    if (pieces && (!vec || F > kPieceMaxL || T > kBufferMaxT)) return false;
    AlphaArgs a{};
    a.out = out; a.in = in; a.filt = filt;
    a.rows = nNeurons;
    a.T = static_cast<int>(T);
    a.L = static_cast<int>(F);
    const double ratio = static_cast<double>(Ts) / static_cast<double>(tau);
    a.a = static_cast<float>(exp(-ratio));
    // (powers of the rounded a, which is what the recursion multiplies by; a lane's segment is units / 16 or one more
    // units long, a unit being a vector or a sample)
    const int64_t perUnit = vec ? 4 : 1, shortest = (vec ? T / 4 : T) / parts;
    a.aSeg[0] = static_cast<float>(pow(static_cast<double>(a.a), static_cast<double>(perUnit * shortest)));
    a.aSeg[1] = static_cast<float>(pow(static_cast<double>(a.a), static_cast<double>(perUnit * (shortest + 1))));
    a.aL = static_cast<float>(pow(static_cast<double>(a.a), static_cast<double>(F)));
    a.scale = static_cast<float>(static_cast<double>(Ts) * static_cast<double>(mult) * exp(1.0) * ratio);
    a.Ts = Ts;
    a.u = u; a.theta = theta; a.tauRho = tauRho; a.gain = gain;
    a.add = add;
    const dim3 grid(static_cast<unsigned>(tiles));
    if (pieces) {
        AlphaPieces pc{};
        pc.H = static_cast<int>((F + 3) / 4 * 4);
        const int64_t lastUnits = (T / 4) % (kPieceT / 4);      // vectors per row in a shorter last piece (0: none)
        const double ad = static_cast<double>(a.a);
        for (int i = 0; i < 5; ++i) pc.aPow[i] = static_cast<float>(pow(ad, 16.0 * static_cast<double>(1 << i)));
        pc.aSegLast[0] = static_cast<float>(pow(ad, 4.0 * static_cast<double>(lastUnits / parts)));
        pc.aSegLast[1] = static_cast<float>(pow(ad, 4.0 * static_cast<double>(lastUnits / parts + 1)));
        const size_t ldsPieces = static_cast<size_t>(R) * (2 * kPieceT + pc.H) * sizeof(float);
#define SLAYER_PIECES_LAUNCH(OFFV)                                                                                      \
        do {                                                                                                           \
            if (u && gateOut) hipLaunchKernelGGL((alpha_psp_pieces_kernel<false, 2, OFFV>), grid, dim3(kWave), ldsPieces, st, a, pc); \
            else if (u) hipLaunchKernelGGL((alpha_psp_pieces_kernel<false, 1, OFFV>), grid, dim3(kWave), ldsPieces, st, a, pc);       \
            else if (causal) hipLaunchKernelGGL((alpha_psp_pieces_kernel<true, 0, OFFV>), grid, dim3(kWave), ldsPieces, st, a, pc);   \
            else hipLaunchKernelGGL((alpha_psp_pieces_kernel<false, 0, OFFV>), grid, dim3(kWave), ldsPieces, st, a, pc);              \
        } while (0)
        switch (pc.H - static_cast<int>(F)) {
            case 0: SLAYER_PIECES_LAUNCH(0); break;
            case 1: SLAYER_PIECES_LAUNCH(1); break;
            case 2: SLAYER_PIECES_LAUNCH(2); break;
            default: SLAYER_PIECES_LAUNCH(3); break;
        }
#undef SLAYER_PIECES_LAUNCH
        return true;
    }
    const size_t lds = static_cast<size_t>(2) * R * T * sizeof(float);
#define SLAYER_ALPHA_LAUNCH(VEC)                                                                                       \
    do {                                                                                                              \
        if (u && gateOut) hipLaunchKernelGGL((alpha_psp_kernel<false, R, 2, VEC>), grid, dim3(kWave), lds, st, a);    \
        else if (u) hipLaunchKernelGGL((alpha_psp_kernel<false, R, 1, VEC>), grid, dim3(kWave), lds, st, a);          \
        else if (causal) hipLaunchKernelGGL((alpha_psp_kernel<true, R, 0, VEC>), grid, dim3(kWave), lds, st, a);      \
        else hipLaunchKernelGGL((alpha_psp_kernel<false, R, 0, VEC>), grid, dim3(kWave), lds, st, a);                 \
    } while (0)
    if (vec) SLAYER_ALPHA_LAUNCH(true);
    else SLAYER_ALPHA_LAUNCH(false);
#undef SLAYER_ALPHA_LAUNCH
    return true;
}

}  // namespace slayer

extern "C" int slayer_psp_alpha_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T, int64_t F,
                                    float tau, float mult, float Ts, int causal, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || F < 1 || !(tau > 0.0f) || !(Ts > 0.0f)) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!out || !in || !filt) return SLAYER_EINVAL;
    if (launch_alpha(out, in, filt, nNeurons, T, F, tau, mult, Ts, causal != 0, nullptr, 0.0f, 1.0f, 0.0f,
                     static_cast<hipStream_t>(stream)))
        return launch_status();
    // the sum over the taps of the given filter
    return causal ? slayer_conv_f32(out, in, filt, nNeurons, T, F, Ts, stream)
                  : slayer_corr_f32(out, in, filt, nNeurons, T, F, Ts, stream);
}

extern "C" int slayer_spike_bwd_psp_alpha_f32(float *gradIn, const float *gradOut, const float *u, const float *filt,
                                              int64_t nNeurons, int64_t T, int64_t F, float tau, float mult, float theta,
                                              float tauRho, float scale, float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || F < 1 || !(tau > 0.0f) || !(Ts > 0.0f) || tauRho == 0.0f) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!gradIn || !gradOut || !u || !filt) return SLAYER_EINVAL;
    if (launch_alpha(gradIn, gradOut, filt, nNeurons, T, F, tau, mult, Ts, false, u, theta, tauRho, scale / tauRho,
                     static_cast<hipStream_t>(stream)))
        return launch_status();
    return slayer_spike_bwd_corr_f32(gradIn, gradOut, u, filt, nNeurons, T, F, theta, tauRho, scale, Ts, stream);
}

extern "C" int slayer_psp_spike_bwd_alpha_f32(float *gradIn, const float *gradPsp, const float *gradSpike, const float *u,
                                              const float *filt, int64_t nNeurons, int64_t T, int64_t F, float tau, float mult,
                                              float theta, float tauRho, float scale, float Ts, void *stream)
{
    using namespace slayer;
    if (nNeurons < 0 || T < 0 || F < 1 || !(tau > 0.0f) || !(Ts > 0.0f) || tauRho == 0.0f) return SLAYER_EINVAL;
    if (nNeurons == 0 || T == 0) return SLAYER_OK;
    if (!gradIn || !gradPsp || !u || !filt) return SLAYER_EINVAL;
    if (launch_alpha(gradIn, gradPsp, filt, nNeurons, T, F, tau, mult, Ts, false, u, theta, tauRho, scale / tauRho,
                     static_cast<hipStream_t>(stream), true, gradSpike))
        return launch_status();
    return SLAYER_EUNSUPPORTED;  // the caller runs slayer_corr_f32, adds and calls slayer_spike_bwd_f32
}

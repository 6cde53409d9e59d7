// Register-window core of the FIR kernels: a lane produces U consecutive outputs of
// Y[m] = sum_i X[m+i] * filt[i] from a window of X that slides through LDS.
#ifndef SLAYER_CSRC_FIR_CORE_H
#define SLAYER_CSRC_FIR_CORE_H

#include "common.h"

namespace slayer {

// Optional gate on the input: the filter then runs over in[n][t] * gain * exp(-|u[n][t] - theta| / tau),
// i.e. the spike function's surrogate gradient applied on the way in (u == nullptr: no gate).
struct FirGate {
    const float *u;
    float theta, tau, gain;
};

// Matrix-core correlation (fir_mfma.hip).  Returns false, launching nothing, for shapes it does not serve.
bool launch_fir_corr_mfma(float *out, const float *in, const float *filt, int64_t rows, int64_t T, int64_t F, float Ts,
                          const FirGate &gate, hipStream_t stream);

// Filter lengths that the matrix-core paths serve (the correlation kernel of fir_mfma.hip and the dense tiles of
// the tiled kernel of fir.hip).
constexpr int kFirMfmaMinTaps = 34, kFirMfmaMaxTaps = 129;

// ---- operands of the bf16 matrix instruction from fp32 numbers (the three-way split that fir_mfma.hip describes) ----
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

struct SplitPlanes {
    uint4_ext hi, mid, lo;  // 8 bf16 each: element e in the lower (even e) or upper half of word e / 2
};

__device__ __forceinline__ SplitPlanes split_bf16(const float (&x)[8])
{
    uint32_t a[8], b[8], cc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        a[e] = __builtin_bit_cast(uint32_t, x[e]);
        const float r1 = x[e] - __builtin_bit_cast(float, a[e] & 0xffff0000u);  // exact
        b[e] = __builtin_bit_cast(uint32_t, r1);
        const float r2 = r1 - __builtin_bit_cast(float, b[e] & 0xffff0000u);  // exact
        cc[e] = __builtin_bit_cast(uint32_t, r2);
    }
    SplitPlanes s;
#pragma unroll
    for (int w = 0; w < 4; ++w) {  // the upper halves of two words into one
        s.hi[w] = __builtin_amdgcn_perm(a[2 * w + 1], a[2 * w], 0x07060302u);
        s.mid[w] = __builtin_amdgcn_perm(b[2 * w + 1], b[2 * w], 0x07060302u);
        s.lo[w] = __builtin_amdgcn_perm(cc[2 * w + 1], cc[2 * w], 0x07060302u);
    }
    return s;
}

__device__ __forceinline__ f32x4 mfma_bf16(const uint4_ext &a, const uint4_ext &b, f32x4 acc)
{
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), acc, 0, 0, 0);
}

// A lane produces U consecutive outputs from a register window of U + 4 samples held as
// NQ = U/4 + 1 16-byte vectors q[].  ROT says which vector currently holds the oldest samples:
// window sample e is component e % 4 of q[(ROT + e / 4) % NQ].  After a 4-tap block the oldest
// vector is replaced by the next one from LDS and ROT advances, so the window slides without any
// register moves once the loops are unrolled.
template <int U, int ROT>
__device__ __forceinline__ void window_of(float (&w)[U + 4], const float4 (&q)[U / 4 + 1])
{
    constexpr int NQ = U / 4 + 1;
#pragma unroll
    for (int v = 0; v < NQ; ++v) {
        const float4 &x = q[(ROT + v) % NQ];
        w[4 * v] = x.x; w[4 * v + 1] = x.y; w[4 * v + 2] = x.z; w[4 * v + 3] = x.w;
    }
}

// taps f0..f3 are filter taps i..i+3; output j, tap s uses window sample j + s
template <int U, int ROT>
__device__ __forceinline__ void fma_block(float (&acc)[U], const float4 (&q)[U / 4 + 1], float f0, float f1,
                                          float f2, float f3)
{
    float w[U + 4];
    window_of<U, ROT>(w, q);
#pragma unroll
    for (int j = 0; j < U; ++j) {
        acc[j] = __builtin_fmaf(w[j + 0], f0, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 1], f1, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 2], f2, acc[j]);
        acc[j] = __builtin_fmaf(w[j + 3], f3, acc[j]);
    }
}

// the last 1..3 taps of a filter whose length is not a multiple of 4
template <int U, int ROT>
__device__ __forceinline__ void fma_rest(float (&acc)[U], const float4 (&q)[U / 4 + 1], const float *__restrict__ f,
                                         int n)
{
    float w[U + 4];
    window_of<U, ROT>(w, q);
    const float f0 = f[0];
    const float f1 = n > 1 ? f[1] : 0.0f;
    const float f2 = n > 2 ? f[2] : 0.0f;
#pragma unroll
    for (int j = 0; j < U; ++j) {
        acc[j] = __builtin_fmaf(w[j], f0, acc[j]);
        if (n > 1) acc[j] = __builtin_fmaf(w[j + 1], f1, acc[j]);
        if (n > 2) acc[j] = __builtin_fmaf(w[j + 2], f2, acc[j]);
    }
}

// blocks B, B+1, .., NQ-1 of one trip of the main loop (NQ blocks = 4 NQ taps per trip)
template <int U, int B>
struct TripBlocks {
    static __device__ __forceinline__ void run(float (&acc)[U], float4 (&q)[U / 4 + 1], const float4 *xq, int qi,
                                               const float *__restrict__ f)
    {
        if constexpr (B < U / 4 + 1) {
            fma_block<U, B>(acc, q, f[4 * B], f[4 * B + 1], f[4 * B + 2], f[4 * B + 3]);
            q[B] = xq[qi + B];
            TripBlocks<U, B + 1>::run(acc, q, xq, qi, f);
        }
    }
};

// up to NQ-1 further whole blocks after the main loop, then the rest; B = blocks done so far
template <int U, int B>
struct TailBlocks {
    static __device__ __forceinline__ void run(float (&acc)[U], float4 (&q)[U / 4 + 1], const float4 *xq, int qi,
                                               const float *__restrict__ f, int left)
    {
        if constexpr (B < U / 4 + 1) {
            if (left >= 4) {
                fma_block<U, B>(acc, q, f[0], f[1], f[2], f[3]);
                q[B] = xq[qi];
                TailBlocks<U, B + 1>::run(acc, q, xq, qi + 1, f + 4, left - 4);
            } else if (left > 0) {
                fma_rest<U, B>(acc, q, f, left);
            }
        }
    }
};

}  // namespace slayer

#endif

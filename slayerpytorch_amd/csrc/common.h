// Shared host/device helpers of libslayer_hip (gfx950 only).
#ifndef SLAYER_CSRC_COMMON_H
#define SLAYER_CSRC_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/slayer_hip.h"

namespace slayer {

constexpr int kWave = 64;  // CDNA wavefront width

// Records a HIP runtime failure for slayer_last_hip_error() and maps it to a status code.
int note_hip_error(hipError_t err);

// Status of the launch that was just enqueued on this thread.
inline int launch_status() { return note_hip_error(hipGetLastError()); }

// Compute units of the current device (256 on MI355X); persistent kernels size their grid by it.
int compute_units();

// True when slayer_force_generic_kernels(1) is in effect.
bool generic_forced();

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// float -> int32 toward zero; saturates at INT32_MIN / INT32_MAX and maps NaN to 0, like the
// hardware conversion, but spelled out so that no out-of-range cast is ever evaluated.
__device__ __forceinline__ int trunc_sat(float x)
{
    if (!(x == x)) return 0;
    if (x >= 2147483648.0f) return 2147483647;
    if (x <= -2147483648.0f) return -2147483647 - 1;
    return static_cast<int>(x);
}

// Number of whole sampling steps in a delay: fp32 quotient truncated toward zero.
__device__ __forceinline__ int delay_steps(float delay, float Ts) { return trunc_sat(delay / Ts); }

// i / d for 0 <= i < 2^24 with a precomputed float reciprocal (estimate plus one correction)
__device__ __forceinline__ void divmod_small(int i, int d, float inv, int &q, int &r)
{
    q = static_cast<int>(static_cast<float>(i) * inv);
    r = i - q * d;
    if (r < 0) { --q; r += d; }
    else if (r >= d) { ++q; r -= d; }
}

// (row, column) = divmod(index, width) advanced incrementally: the work index grows by 256 per
// trip, so the pair moves by (256 / width, 256 % width) with one carry.
struct RowCol {
    int r, c;
    __device__ __forceinline__ void init(int index, int width, float inv) { divmod_small(index, width, inv, r, c); }
    __device__ __forceinline__ void advance(int dr, int dc, int width)
    {
        r += dr;
        c += dc;
        if (c >= width) { c -= width; ++r; }
    }
};

// Surrogate gradient of the spike function at membrane potential u: gain * exp(-|u - theta| / tau)
// with gain = scale / tau.
__device__ __forceinline__ float spike_pdf(float u, float theta, float tau, float gain)
{
    return gain * expf(-fabsf(u - theta) / tau);
}

// Synchronisation inside a work-group that is a single wavefront.  LDS executes the accesses of
// one wavefront in program order, so data written by one lane is visible to the other lanes of
// the same wavefront in any later instruction; all that is needed is to keep the compiler from
// moving LDS accesses across this point.  Unlike __syncthreads() it does not wait for the
// wavefront's outstanding global loads and stores, which is the point: prefetches and stores
// stay in flight across it.
__device__ __forceinline__ void wave_sync()
{
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Division of a 32-bit unsigned number by a constant chosen on the host (Granlund-Montgomery):
// q = (t + ((n - t) >> s1)) >> s2 with t = mulhi(n, m).  Exact for every n and every d >= 1.
struct FastDiv {
    uint32_t d, m, s1, s2;
};

inline FastDiv make_fastdiv(uint32_t d)
{
    FastDiv f;
    f.d = d;
    uint32_t l = 0;
    while (l < 32 && (static_cast<uint64_t>(1) << l) < d) ++l;  // ceil(log2 d)
    f.m = static_cast<uint32_t>(((static_cast<uint64_t>(1) << 32) * ((static_cast<uint64_t>(1) << l) - d)) / d + 1);
    f.s1 = l < 1 ? l : 1;
    f.s2 = l > 0 ? l - 1 : 0;
    return f;
}

__device__ __forceinline__ uint32_t fastdiv(uint32_t n, const FastDiv &f)
{
    const uint32_t t = __umulhi(n, f.m);
    return (t + ((n - t) >> f.s1)) >> f.s2;
}

// Work-groups are handed to the GPU's 8 accelerator dies (XCDs, each with its own L2) round-robin by
// index: group b runs on die b % 8.  Kernels whose neighbouring groups read the same data (filter
// windows that overlap, operands shared between tiles) would make every die fetch all of it.  This
// maps the hardware index to a logical one so that each die owns one contiguous range of logical
// indices: die x gets the k-th index of its range for its k-th group.
__device__ __forceinline__ uint32_t xcd_contiguous(uint32_t b, uint32_t n)
{
    constexpr uint32_t kDies = 8;
    const uint32_t per = n / kDies, rem = n % kDies;  // die x owns per + (x < rem) indices
    const uint32_t x = b % kDies, k = b / kDies;
    return x * per + (x < rem ? x : rem) + k;
}

// ---- buffer addressing -------------------------------------------------------------------------
// address = base (128-bit descriptor in scalar registers) + per-lane byte offset (one vector
// register) + wave-uniform byte offset (scalar register).  Lets a wave touch many rows of a tile
// without a 64-bit address register per access.  Both offsets are 32 bit: kernels that use it
// keep tiles below 2 GiB (rows of at most kBufferMaxT samples).
typedef __amdgpu_buffer_rsrc_t BufferRsrc;
constexpr int64_t kBufferMaxT = 1 << 22;

// The same with a range check: accesses at byte offsets >= bytes read zeros / are dropped.
__device__ __forceinline__ BufferRsrc make_buffer(const void *base, int bytes)
{
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

__device__ __forceinline__ BufferRsrc make_buffer(const void *base)
{
    // raw buffer, no stride/swizzle, 32-bit data format; range = the whole 32-bit offset space
    // (validity of every access is established by the caller's own predicates)
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, 0x7fffffff, 0x00020000);
}

// Cache policy of the streaming accesses: every tensor on this path is read once and written
// once per kernel, so the "non-temporal" hint keeps them from displacing each other in L2
// (measured on MI355X: a 16-byte-per-lane copy runs at 6.5 TB/s with the hint, 6.0 without).
constexpr int kStream = 2;  // "nt" bit of the buffer instruction's cache-policy field
// Loads of kernels that walk along rows whose input is typically another kernel's recent output or a tensor that is
// read again soon (the PSP recursion, the Loihi neuron) keep the default policy.  Measured with plain copies of the
// walking pattern: the hint on loads gains nothing on tensors beyond the 256 MB last-level cache (1 GB moved: 202 us
// with the hint on stores only, 205 us on both) and costs a third when the input fits that cache and was touched
// recently (262 MB moved: 36 us against 54 us), because the hint keeps it from being found there.  Stores keep the
// hint at every size; kernels whose loads are one flat stream keep it on loads too (6 % on large tensors).
constexpr int kCached = 0;

template <int POLICY = kStream>
__device__ __forceinline__ float buffer_load(BufferRsrc b, int laneBytes, int uniformBytes)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(b, laneBytes, uniformBytes, POLICY));
}

typedef float float4_ext __attribute__((ext_vector_type(4)));
typedef unsigned int uint4_ext __attribute__((ext_vector_type(4)));

// Offset that lies outside every buffer made by make_buffer(): a load from it returns zeros and a
// store to it is dropped by the hardware's range check.  Masking accesses this way instead of
// branching around them keeps the number of memory instructions between two points fixed, so
// the compiler can wait for "all but the last N" (s_waitcnt vmcnt(N)) instead of for everything.
constexpr int kOutOfRange = static_cast<int>(0x80000000u);

__device__ __forceinline__ int masked_offset(bool valid, int bytes) { return valid ? bytes : kOutOfRange; }

template <int POLICY = kStream>
__device__ __forceinline__ float4 buffer_load4(BufferRsrc b, int laneBytes, int uniformBytes)
{
    const uint4_ext x = __builtin_amdgcn_raw_buffer_load_b128(b, laneBytes, uniformBytes, POLICY);
    const float4_ext f = __builtin_bit_cast(float4_ext, x);
    return make_float4(f.x, f.y, f.z, f.w);
}

template <int POLICY = kStream>
__device__ __forceinline__ void buffer_store4(BufferRsrc b, int laneBytes, int uniformBytes, float4 v)
{
    const float4_ext f = {v.x, v.y, v.z, v.w};
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4_ext, f), b, laneBytes, uniformBytes, POLICY);
}

template <int POLICY = kStream>
__device__ __forceinline__ void buffer_store(BufferRsrc b, int laneBytes, int uniformBytes, float x)
{
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, x), b, laneBytes, uniformBytes, POLICY);
}

}  // namespace slayer

#endif

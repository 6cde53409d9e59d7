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

}  // namespace slayer

#endif

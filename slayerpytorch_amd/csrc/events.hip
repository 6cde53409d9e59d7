// Spike event files to spike tensors on the device: decoding of the packed event layouts of
// src/spikeFileIO.py (read1Dspikes :162-184, read2Dspikes :233-259, read3Dspikes :296-321) and the
// binning of event.toSpikeTensor (:66-144), so that a data loader ships a few kilobytes of events
// per sample to the GPU instead of a dense (C, H, W, T) tensor.
//
// Integer and byte work; the one floating-point step, bin = rint((t in ms) / samplingTime), is done in
// IEEE double precision exactly like numpy does it, so the result is bit-identical to the host code.
#include "common.h"

namespace slayer {

struct Event {
    int x, y, p, tUs;
};

// One packed event; FORMAT 1: 16-bit neuron id, 1-bit polarity, 23-bit time; 2: 8-bit x, 8-bit y,
// 1-bit polarity, 23-bit time; 3: 12-bit x, 12-bit y, 8-bit channel, 24-bit time (big-endian fields).
template <int FORMAT>
__device__ __forceinline__ Event decode_event(const uint8_t *b)
{
    Event e;
    if (FORMAT == 3) {
        e.x = (b[0] << 4) | (b[1] >> 4);
        e.y = b[2] | ((b[1] & 0x0F) << 8);
        e.p = b[3];
        e.tUs = (b[4] << 16) | (b[5] << 8) | b[6];
    } else {
        e.x = FORMAT == 1 ? ((b[0] << 8) | b[1]) : b[0];
        e.y = FORMAT == 1 ? 0 : b[1];
        e.p = b[2] >> 7;
        e.tUs = ((b[2] << 16) | (b[3] << 8) | b[4]) & 0x7FFFFF;
    }
    return e;
}

struct BinGeom {
    int C, H, W, T, mode;
    double samplingTime;
    float value;  // (float)(1 / samplingTime)
};

// Writes one event into a [C][H][W][T] tensor.  Every event of a bin writes the same value (the
// constant in OR mode, the untouched `base` value plus the constant in SUM mode), so events that
// share a bin need no ordering.
__device__ __forceinline__ void bin_event(float *tensor, const float *base, int x, int y, int p, double tMs,
                                          double shift, const BinGeom &g)
{
    const double bin = rint(tMs / g.samplingTime) - shift;
    if (!(bin >= 0.0 && bin < static_cast<double>(g.T))) return;  // also drops NaN
    if (static_cast<unsigned>(x) >= static_cast<unsigned>(g.W) || static_cast<unsigned>(y) >= static_cast<unsigned>(g.H) ||
        static_cast<unsigned>(p) >= static_cast<unsigned>(g.C))
        return;
    const int64_t idx = ((static_cast<int64_t>(p) * g.H + y) * g.W + x) * g.T + static_cast<int64_t>(bin);
    tensor[idx] = g.mode == 0 ? g.value : base[idx] + g.value;
}

// One work-group per (sample, slice of its events).  The polarity of a sample's events is shifted so
// that its minimum over the WHOLE sample is 0 (event.__init__, src/spikeFileIO.py:33), so every
// work-group first scans the polarity field of all events of its sample.
// table[s] = {first byte of the sample in `bytes`, number of events, time shift in bins}.
template <int FORMAT>
__global__ __launch_bounds__(256) void bin_packed_events_kernel(float *tensor, const float *base,
                                                                const uint8_t *__restrict__ bytes,
                                                                const int64_t *__restrict__ table, int64_t nBytes,
                                                                int slices, BinGeom g)
{
    constexpr int kBytes = FORMAT == 3 ? 7 : 5;
    __shared__ int wmin[4];
    const int s = blockIdx.x / slices, slice = blockIdx.x - s * slices;
    const int64_t first = table[3 * s], nEvents = table[3 * s + 1], shift = table[3 * s + 2];
    const uint8_t *ev = bytes + first;
    // a table entry that does not lie inside the byte buffer is skipped as a whole
    if (first < 0 || nEvents < 0 || nEvents > (nBytes - first) / kBytes || first > nBytes) return;

    int pmin = 255;
    for (int64_t e = threadIdx.x; e < nEvents; e += 256) {
        const int p = FORMAT == 3 ? ev[e * kBytes + 3] : (ev[e * kBytes + 2] >> 7);
        pmin = min(pmin, p);
    }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) pmin = min(pmin, __shfl_xor(pmin, off, kWave));
    if ((threadIdx.x & (kWave - 1)) == 0) wmin[threadIdx.x / kWave] = pmin;
    __syncthreads();
    pmin = min(min(wmin[0], wmin[1]), min(wmin[2], wmin[3]));

    const int64_t plane = static_cast<int64_t>(g.C) * g.H * g.W * g.T;
    float *dst = tensor + s * plane;
    const float *src = base + s * plane;
    const int64_t per = (nEvents + slices - 1) / slices;
    const int64_t end = min(nEvents, (slice + 1) * per);
    for (int64_t e = slice * per + threadIdx.x; e < end; e += 256) {
        const Event v = decode_event<FORMAT>(ev + e * kBytes);
        bin_event(dst, src, v.x, v.y, v.p - pmin, static_cast<double>(v.tUs) / 1000.0, static_cast<double>(shift), g);
    }
}

// Events that are already decoded (x, y, p as int32, t in ms as double), one sample.
__global__ __launch_bounds__(256) void bin_events_kernel(float *tensor, const float *base, const int32_t *__restrict__ x,
                                                         const int32_t *__restrict__ y, const int32_t *__restrict__ p,
                                                         const double *__restrict__ tMs, int64_t nEvents, double shift,
                                                         BinGeom g)
{
    const int64_t e = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (e >= nEvents) return;
    bin_event(tensor, base, x[e], y ? y[e] : 0, p[e], tMs[e], shift, g);
}

static int make_geom(BinGeom &g, int32_t C, int32_t H, int32_t W, int32_t T, double samplingTime, int32_t mode)
{
    if (C < 0 || H < 0 || W < 0 || T < 0 || (mode != 0 && mode != 1)) return SLAYER_EINVAL;
    if (!(samplingTime > 0.0)) return SLAYER_EINVAL;
    g = BinGeom{C, H, W, T, mode, samplingTime, static_cast<float>(1.0 / samplingTime)};
    return SLAYER_OK;
}

}  // namespace slayer

extern "C" int slayer_bin_packed_events_f32(float *tensor, const float *base, const uint8_t *bytes, int64_t nBytes,
                                            const int64_t *sampleTable, int64_t nSamples, int64_t maxEvents,
                                            int32_t format, int32_t C, int32_t H, int32_t W, int32_t T,
                                            double samplingTime, int32_t mode, void *stream)
{
    using namespace slayer;
    BinGeom g;
    const int status = make_geom(g, C, H, W, T, samplingTime, mode);
    if (status != SLAYER_OK) return status;
    if (format < 1 || format > 3 || nSamples < 0 || maxEvents < 0 || nBytes < 0) return SLAYER_EINVAL;
    if (nSamples == 0 || maxEvents == 0 || static_cast<int64_t>(C) * H * W * T == 0) return SLAYER_OK;
    if (!tensor || !bytes || !sampleTable) return SLAYER_EINVAL;
    if (mode == 1 && (!base || base == tensor)) return SLAYER_EINVAL;
    if (!base) base = tensor;
    // slices per sample: about 2048 events per work-group
    int64_t slices = ceil_div(maxEvents, 2048);
    if (slices > 1024) slices = 1024;
    if (nSamples * slices >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    const dim3 grid(static_cast<unsigned>(nSamples * slices));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int sl = static_cast<int>(slices);
    if (format == 1) hipLaunchKernelGGL(bin_packed_events_kernel<1>, grid, dim3(256), 0, st, tensor, base, bytes, sampleTable, nBytes, sl, g);
    else if (format == 2) hipLaunchKernelGGL(bin_packed_events_kernel<2>, grid, dim3(256), 0, st, tensor, base, bytes, sampleTable, nBytes, sl, g);
    else hipLaunchKernelGGL(bin_packed_events_kernel<3>, grid, dim3(256), 0, st, tensor, base, bytes, sampleTable, nBytes, sl, g);
    return launch_status();
}

extern "C" int slayer_bin_events_f32(float *tensor, const float *base, const int32_t *x, const int32_t *y,
                                     const int32_t *p, const double *tMs, int64_t nEvents, int64_t timeShift,
                                     int32_t C, int32_t H, int32_t W, int32_t T, double samplingTime,
                                     int32_t mode, void *stream)
{
    using namespace slayer;
    BinGeom g;
    const int status = make_geom(g, C, H, W, T, samplingTime, mode);
    if (status != SLAYER_OK) return status;
    if (nEvents < 0) return SLAYER_EINVAL;
    if (nEvents == 0 || static_cast<int64_t>(C) * H * W * T == 0) return SLAYER_OK;
    if (!tensor || !x || !p || !tMs) return SLAYER_EINVAL;
    if (mode == 1 && (!base || base == tensor)) return SLAYER_EINVAL;
    if (!base) base = tensor;
    const int64_t blocks = ceil_div(nEvents, 256);
    if (blocks >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    hipLaunchKernelGGL(bin_events_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       tensor, base, x, y, p, tMs, nEvents, static_cast<double>(timeShift), g);
    return launch_status();
}

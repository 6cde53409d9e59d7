// Fully connected synapse on sparse input, event by event.
//
// The dense layer of the reference (slayer._denseLayer, src/slayer.py:393-440) is a 3-D convolution whose
// kernel spans the whole (C, H, W) extent of its input: per batch item one matrix product
// out[O x T] = W[O x K] * x[K x T], K = C*H*W, with the weight gradient
//
//   gradW[o][k] = sum over n, t of gradOut[n][o][t] * x[n][k][t].
//
// The input is a spike tensor: a few per cent of x is non-zero, and a sum that skips the zeros does a
// few per cent of the work.  For the weight gradient the rows of x are contiguous in t, so a wavefront
// that owns an input channel reads them as they are; the output channels o are on the lanes, so what an
// event fetches is one contiguous row of O floats of the transposed gradient gT[n][t][O] (transposed here
// first; it is small next to x).  The sum runs over the events in ascending (n, t), so the result does
// not depend on scheduling.  The product is the same sum with the roles changed: x transposed to
// [N][T][K] makes a column (n, t) a contiguous row, whose events fetch rows of the transposed weights
// wT[K][O]; the result [N][T][O] is transposed back.  Both are the dense products up to the order of the
// additions (and up to the 0 * inf = NaN terms that a dense product has for non-finite factors).  The work
// is proportional to the number of events: for inputs that are not sparse the matrix product of a
// library is the better choice, and the caller decides.
#include "common.h"

namespace slayer {

__device__ __forceinline__ float cached_load(BufferRsrc b, int laneBytes, int uniformBytes)
{
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(b, laneBytes, uniformBytes, 0));
}

struct DenseEventWgradArgs {
    float *part;  // [slices][K][O]
    const float *x, *gT;
    int N, K, O, T;
    int blocksPerItem;   // ceil(T / 64)
    int blocksPerSlice;  // blocks of 64 samples per slice
};

constexpr int kDeBlocks = 8;  // blocks of 64 samples whose events are listed together
constexpr int kDeBatch = 8;   // events whose rows are in flight together

// One wavefront per (input channel k, slice of the batch's samples).  It reads the channel's samples 512 at a
// time (8 loads in flight), lists the non-zero ones - value and byte offset of the row gT[n][t][:] - in
// LDS in ascending (n, t), and adds value * row to its accumulators (lane l the output channels l + 64 r)
// eight events at a time, whatever block they came from: at 1-2 % non-zero inputs a block of 64 samples
// holds about one event, and taking the blocks one by one left every event's fetch a round trip of its
// own.  part[slice][k][:] takes the sums.  Slices exist so that layers with few input channels still fill
// the GPU; transpose_sum_kernel adds them up.
template <int OR>
__global__ __launch_bounds__(64) void dense_events_wgrad_kernel(DenseEventWgradArgs p)
{
    __shared__ float value[kDeBlocks * 64];
    __shared__ int rowBytes[kDeBlocks * 64];
    const int lane = threadIdx.x;
    const int k = blockIdx.x % p.K, slice = blockIdx.x / p.K;  // channels of one slice run together: they share gT rows
    const int blocks = p.N * p.blocksPerItem;
    const int b0 = slice * p.blocksPerSlice;
    const int b1 = min(b0 + p.blocksPerSlice, blocks);
    const BufferRsrc bg = make_buffer(p.gT, p.N * p.T * p.O * 4);

    float acc[OR];
    int oBytes[OR];
#pragma unroll
    for (int r = 0; r < OR; ++r) {
        acc[r] = 0.0f;
        oBytes[r] = masked_offset(lane + 64 * r < p.O, (lane + 64 * r) * 4);
    }

    for (int b = b0; b < b1; b += kDeBlocks) {
        float v[kDeBlocks];
        int sample[kDeBlocks];  // n * T + t of this lane's sample of block j
#pragma unroll
        for (int j = 0; j < kDeBlocks; ++j) {
            const int bj = min(b + j, b1 - 1);
            const int n = bj / p.blocksPerItem;
            const int t0 = (bj - n * p.blocksPerItem) * 64;
            // one row of x: accesses past its end read zeros (and so does a block past the slice's last)
            const BufferRsrc bx = make_buffer(p.x + (static_cast<int64_t>(n) * p.K + k) * p.T, p.T * 4);
            v[j] = buffer_load(bx, masked_offset(b + j < b1, (t0 + lane) * 4), 0);
            sample[j] = n * p.T + t0 + lane;
        }
        int m = 0;  // events of these blocks
#pragma unroll
        for (int j = 0; j < kDeBlocks; ++j) {
            const bool nz = v[j] != 0.0f;
            const uint64_t mask = __builtin_amdgcn_ballot_w64(nz);
            const int at = m + __builtin_amdgcn_mbcnt_hi(static_cast<uint32_t>(mask >> 32), __builtin_amdgcn_mbcnt_lo(static_cast<uint32_t>(mask), 0));
            if (nz) {
                value[at] = v[j];
                rowBytes[at] = sample[j] * p.O * 4;
            }
            m += __builtin_popcountll(mask);
        }
        wave_sync();
        for (int e = 0; e < m; e += kDeBatch) {
            float val[kDeBatch], g[kDeBatch][OR];
#pragma unroll
            for (int i = 0; i < kDeBatch; ++i) {
                // entries past the end of the list are stale: row 0 with value 0 instead
                const bool live = e + i < m;
                const int at = (e + i) & (kDeBlocks * 64 - 1);
                val[i] = live ? value[at] : 0.0f;
                const int row = __builtin_amdgcn_readfirstlane(live ? rowBytes[at] : 0);
#pragma unroll
                for (int r = 0; r < OR; ++r) g[i][r] = cached_load(bg, oBytes[r], row);
            }
#pragma unroll
            for (int i = 0; i < kDeBatch; ++i)
#pragma unroll
                for (int r = 0; r < OR; ++r) acc[r] = fmaf(val[i], g[i][r], acc[r]);
        }
        wave_sync();  // the lists are rewritten by the next round
    }

    float *dst = p.part + (static_cast<int64_t>(slice) * p.K + k) * p.O;
#pragma unroll
    for (int r = 0; r < OR; ++r)
        if (lane + 64 * r < p.O) dst[lane + 64 * r] = acc[r];
}

// dst[b][c][r] = sum over s of src[b][s][r][c], matrix (b, s) of src starting b * batchStride + s * sliceStride
// floats in: tiles of 32 x 32 (64 x 64 for large single matrices: 256 bytes of a row at a time) through LDS, so
// that both sides are read and written along their rows.
// Transposes gradients, inputs and weights (S = 1) and adds and transposes the slices of a result.
template <int TILE>
__global__ __launch_bounds__(256) void transpose_sum_kernel(float *__restrict__ dst, const float *__restrict__ src,
                                                            int S, int R, int C, int64_t batchStride, int64_t sliceStride)
{
    __shared__ float tile[TILE][TILE + 1];
    constexpr int ROWS = 256 / TILE;  // rows of the tile that the 256 threads cover at a time
    const int x = threadIdx.x % TILE, y = threadIdx.x / TILE;
    const int c0 = blockIdx.x * TILE, r0 = blockIdx.y * TILE;
    const int64_t matrix = static_cast<int64_t>(R) * C;
    const float *from = src + static_cast<int64_t>(blockIdx.z) * batchStride;
    float v[TILE / ROWS];
#pragma unroll
    for (int j = 0; j < TILE / ROWS; ++j) v[j] = 0.0f;
    for (int s = 0; s < S; ++s) {  // (the loads of a slice in flight together)
#pragma unroll
        for (int j = 0; j < TILE / ROWS; ++j) {
            const int r = r0 + y + ROWS * j, c = c0 + x;
            v[j] += (r < R && c < C) ? from[s * sliceStride + static_cast<int64_t>(r) * C + c] : 0.0f;
        }
    }
#pragma unroll
    for (int j = 0; j < TILE / ROWS; ++j) tile[y + ROWS * j][x] = v[j];
    __syncthreads();
    float *to = dst + static_cast<int64_t>(blockIdx.z) * matrix;
#pragma unroll 4
    for (int j = 0; j < TILE / ROWS; ++j) {
        const int c = c0 + y + ROWS * j, r = r0 + x;
        if (r < R && c < C) to[static_cast<int64_t>(c) * R + r] = tile[x][y + ROWS * j];
    }
}

}  // namespace slayer

namespace {

// Everything the kernel addresses with 32-bit byte offsets: gT, one row of x.
bool dense_events_fits(int64_t N, int64_t K, int64_t O, int64_t T)
{
    const int64_t lim = (1LL << 31) - 64;
    return N < (1LL << 24) && N * O * T * 4 < lim && T * 4 < lim;
}

int64_t dense_events_slices(int64_t N, int64_t K, int64_t O, int64_t T)
{
    using namespace slayer;
    if (N <= 0 || K <= 0 || O <= 0 || T <= 0) return 0;
    const int64_t blocks = N * ceil_div(T, 64);
    // about eight wavefronts per SIMD of the whole GPU, each with at least 16 blocks of 64 samples
    const int64_t want = ceil_div(static_cast<int64_t>(compute_units()) * 32, K);
    const int64_t most = ceil_div(blocks, 16);
    int64_t slices = want < most ? want : most;
    if (slices < 1) slices = 1;
    const int64_t per = ceil_div(blocks, slices);
    return ceil_div(blocks, per);
}

// dst[b][c][r] = sum_s src[...][r][c] (see transpose_sum_kernel); false when an extent does not fit a grid
bool launch_transpose_sum(float *dst, const float *src, int64_t B, int64_t S, int64_t R, int64_t C, int64_t batchStride,
                          int64_t sliceStride, hipStream_t st)
{
    using namespace slayer;
    if (B > 65535 || ceil_div(R, 32) > 65535 || ceil_div(C, 32) >= (1LL << 31) || R >= (1LL << 31) || C >= (1LL << 31)) return false;
    if (S == 1 && R * C >= (1LL << 19))
        hipLaunchKernelGGL(transpose_sum_kernel<64>,
                           dim3(static_cast<unsigned>(ceil_div(C, 64)), static_cast<unsigned>(ceil_div(R, 64)), static_cast<unsigned>(B)),
                           dim3(256), 0, st, dst, src, static_cast<int>(S), static_cast<int>(R), static_cast<int>(C), batchStride, sliceStride);
    else
        hipLaunchKernelGGL(transpose_sum_kernel<32>,
                           dim3(static_cast<unsigned>(ceil_div(C, 32)), static_cast<unsigned>(ceil_div(R, 32)), static_cast<unsigned>(B)),
                           dim3(256), 0, st, dst, src, static_cast<int>(S), static_cast<int>(R), static_cast<int>(C), batchStride, sliceStride);
    return true;
}

// part[s][k][o] = sum over the non-zero x[n][k][t] of slice s of x[n][k][t] * rows[n][t][o]; returns the number of slices
// (0: the extents do not fit)
int64_t launch_events(float *part, const float *rows, const float *x, int64_t N, int64_t K, int64_t O, int64_t T, hipStream_t st)
{
    using namespace slayer;
    const int64_t slices = dense_events_slices(N, K, O, T);
    DenseEventWgradArgs p;
    p.part = part; p.x = x; p.gT = rows;
    p.N = static_cast<int>(N); p.K = static_cast<int>(K); p.O = static_cast<int>(O); p.T = static_cast<int>(T);
    p.blocksPerItem = static_cast<int>(ceil_div(T, 64));
    const int64_t blocks = N * p.blocksPerItem;
    if (blocks >= (1LL << 31) || slices * K >= (1LL << 26) || K >= (1LL << 31)) return 0;
    p.blocksPerSlice = static_cast<int>(ceil_div(blocks, slices));
    const dim3 grid(static_cast<unsigned>(slices * K));
    const int perLane = static_cast<int>(ceil_div(O, 64));
    if (perLane <= 1) hipLaunchKernelGGL((dense_events_wgrad_kernel<1>), grid, dim3(64), 0, st, p);
    else if (perLane <= 2) hipLaunchKernelGGL((dense_events_wgrad_kernel<2>), grid, dim3(64), 0, st, p);
    else if (perLane <= 4) hipLaunchKernelGGL((dense_events_wgrad_kernel<4>), grid, dim3(64), 0, st, p);
    else if (perLane <= 8) hipLaunchKernelGGL((dense_events_wgrad_kernel<8>), grid, dim3(64), 0, st, p);
    else hipLaunchKernelGGL((dense_events_wgrad_kernel<16>), grid, dim3(64), 0, st, p);
    return slices;
}

}  // namespace

extern "C" int64_t slayer_dense_events_grad_weight_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T)
{
    if (N <= 0 || K <= 0 || O <= 0 || T <= 0) return 0;
    // the transposed gradient [N][T][O], then the slices [slices][K][O]
    return (N * T * O + dense_events_slices(N, K, O, T) * K * O) * 4;
}

extern "C" int slayer_dense_events_grad_weight_f32(float *gradW, const float *gradOut, const float *x,
                                                   float *workspace, int64_t N, int64_t K, int64_t O, int64_t T,
                                                   void *stream)
{
    using namespace slayer;
    if (N < 0 || K < 0 || O < 0 || T < 0) return SLAYER_EINVAL;
    if (K == 0 || O == 0) return SLAYER_OK;
    if (!gradW) return SLAYER_EINVAL;
    if (N > 0 && T > 0 && (!gradOut || !x || !workspace)) return SLAYER_EINVAL;
    if (!dense_events_fits(N, K, O, T) || O > 64 * 16 || K * O >= (1LL << 31) || N > 65535 || ceil_div(K, 32) > 65535)
        return SLAYER_EUNSUPPORTED;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (N == 0 || T == 0) {  // no samples: the gradient is zero (the sum over no slices)
        launch_transpose_sum(gradW, gradW, 1, 0, K, O, 0, 0, st);
        return launch_status();
    }
    const int64_t slices = dense_events_slices(N, K, O, T);
    if (slices * K >= (1LL << 26) || N * ceil_div(T, 64) >= (1LL << 31)) return SLAYER_EUNSUPPORTED;
    float *gT = workspace, *part = workspace + N * T * O;
    // gT[n][t][o] = gradOut[n][o][t]
    launch_transpose_sum(gT, gradOut, N, 1, O, T, O * T, 0, st);
    launch_events(part, gT, x, N, K, O, T, st);
    // gradW[o][k] = sum over the slices of part[s][k][o]
    launch_transpose_sum(gradW, part, 1, slices, K, O, 0, K * O, st);
    return launch_status();
}

/* The forward product of the same layer on the same kernel: with the input transposed to xT[n][t][k], a column
 * (n, t) of x is a row whose events fetch rows of the transposed weight matrix wT[k][o]. */
extern "C" int64_t slayer_dense_events_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T)
{
    if (N <= 0 || K <= 0 || O <= 0 || T <= 0) return 0;
    // xT [N][T][K], wT [K][O], the slices [slices][N * T][O]
    return (N * T * K + K * O + dense_events_slices(1, N * T, O, K) * N * T * O) * 4;
}

extern "C" int slayer_dense_events_f32(float *out, const float *x, const float *weight, float *workspace, int64_t N,
                                       int64_t K, int64_t O, int64_t T, void *stream)
{
    using namespace slayer;
    if (N < 0 || K < 0 || O < 0 || T < 0) return SLAYER_EINVAL;
    if (N == 0 || O == 0 || T == 0) return SLAYER_OK;
    if (!out) return SLAYER_EINVAL;
    if (K > 0 && (!x || !weight || !workspace)) return SLAYER_EINVAL;
    const int64_t lim = (1LL << 31) - 64;
    if (O > 64 * 16 || O * K * 4 >= lim || K * 4 >= lim || N > 65535 || N * T >= (1LL << 31) || ceil_div(K, 32) > 65535 ||
        ceil_div(T, 32) > 65535 || ceil_div(O, 32) > 65535)
        return SLAYER_EUNSUPPORTED;
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (K == 0) {  // no inputs: zeros (the sum over no slices)
        launch_transpose_sum(out, out, N, 0, T, O, O * T, 0, st);
        return launch_status();
    }
    const int64_t slices = dense_events_slices(1, N * T, O, K);
    if (slices * N * T >= (1LL << 26)) return SLAYER_EUNSUPPORTED;
    float *xT = workspace, *wT = xT + N * T * K, *part = wT + K * O;
    launch_transpose_sum(xT, x, N, 1, K, T, K * T, 0, st);        // xT[n][t][k] = x[n][k][t]
    launch_transpose_sum(wT, weight, 1, 1, O, K, 0, 0, st);       // wT[k][o] = weight[o][k]
    // part[s][(n, t)][o] = sum over the non-zero xT[(n, t)][k] of slice s of xT * wT[k][o]: one batch item of N * T rows
    launch_events(part, wT, xT, 1, N * T, O, K, st);
    // out[n][o][t] = sum over the slices of part[s][n * T + t][o]
    launch_transpose_sum(out, part, N, slices, T, O, T * O, N * T * O, st);
    return launch_status();
}

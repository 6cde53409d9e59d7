// The fully connected synapse as one kernel, for layers whose reduction axis is short (up to 224 inputs per launch):
//
//     out[n][o][t] (+)= sum_{k < K} W[o][k] * x[n][k][t]            W[o][k] = w[o * wRow + k * wCol]
//
// i.e. per batch item the matrix product W (O x K) * x[n] (K x T) with time innermost, as the tensors already are.
// With wRow = K, wCol = 1 this is the layer's forward pass (the reference: a 3-D convolution whose kernel spans the
// whole (C, H, W) extent, src/slayer.py:393-440); with wRow = 1, wCol = K' on the weight of a layer with K' inputs it
// is the input gradient W^T * gradOut.
//
// The product runs on bf16 matrix instructions over a three-way split of both operands (fir_mfma.hip describes the
// split and its error: every fp32 number is hi + mid + lo exactly, six of the nine partial products are kept, each
// exact in the fp32 accumulator; within a few 1e-7 of sum |W||x|).  A spike tensor - values 0 and 1/Ts - is its own
// hi part whenever 1/Ts has at most 8 significant bits (Ts = 1): a tile whose mid and lo parts are all zero, found
// while it is staged, takes only the three products with W's parts.
//
// A work-group of 8 wavefronts walks over tiles of 32 time samples of one batch item.  Wavefront w owns outputs
// 32 w .. 32 w + 31 and keeps their rows of W, split, in registers for the whole launch (12 registers per 32 inputs
// and 16 outputs: 168 at 224 inputs, which is why a launch takes no more).  The tiles of x travel from memory
// straight into a ring of three raw tiles in LDS (buffer_load ... lds: no registers, so the loads of two tiles ahead
// can be in flight during the work on this one; a wavefront's instruction moves 8 rows of 128 bytes, lane l writing
// its 16 bytes at 16 l).  A tile is then split on its way from the ring into three planes [t][k] of bf16, so that a
// lane's operand of v_mfma_f32_16x16x32_bf16 - 8 consecutive k for one t - is one 16-byte read; the row pitch
// (64 KC + 16 bytes) spreads the 16 rows of a read over the banks.  Two barriers per tile: the planes are free
// (everybody has finished the tile before) and the tile has arrived; the planes are written.  The compiler does not
// know that those loads write LDS: the wait for a tile's loads is written out, with the number of memory
// instructions that were issued after them.  The order of the inputs within a plane is a fixed permutation (the
// reduction does not care): inputs k and k + 8 share a word, which lets the lane that splits a pair read both rows
// with the same lane-contiguous pattern the loads wrote.  Lane (c = lane % 16, h = lane / 16) ends up with
// out[o = 16 j + c][t = 16 tt + 4h .. + 3] in its accumulators: one 16-byte store per tile of 16 x 16.
//
// Samples and weights are taken to be finite (the split of an infinity is not).
#include "../../include/slayer_hip.h"
#include "common.h"
#include "fir_core.h"

namespace slayer {

constexpr int kDenseTileT = 32;      // time samples per tile
constexpr int kDenseWaves = 8;       // wavefronts per work-group, 32 outputs each
constexpr int kDenseMaxChunks = 7;   // chunks of 32 inputs per launch
constexpr int kDenseRing = 2;        // raw tiles in LDS

struct DenseRowsArgs {
    float *out;
    const float *x;
    const uint4_ext *wParts;   // W, split, in the order the wavefronts keep it (dense_rows_split_weights_kernel)
    int N, O, K, T;
    int64_t xItem;        // floats between the batch items of x (the launch may see only some of an item's rows)
    int accumulate;       // add to out instead of overwriting it
    int tilesPerItem;
    uint32_t tiles;
};

// s_waitcnt for "at most n vector memory instructions outstanding" and nothing else
template <int N>
__device__ __forceinline__ void wait_vmem()
{
    static_assert(N >= 0 && N < 64, "vmcnt has 6 bits");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (15 << 8) | ((N >> 4) << 14));
}

// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at ldsAddr + 16 l (ldsAddr: the same in all
// lanes).  Written out as the instruction itself: the compiler makes every LDS read that follows the builtin form wait
// for all of them (it cannot tell which part of LDS they fill), which would leave no tile in flight during the work on
// another; it does not count these among the outstanding memory instructions, so the waits it inserts for others
// can only turn out longer than needed, never shorter.
typedef int int4_ext __attribute__((ext_vector_type(4)));
__device__ __forceinline__ int4_ext make_descriptor(const void *base, int bytes)
{
    const uint64_t a = reinterpret_cast<uint64_t>(base);
    const int4_ext d = {static_cast<int>(a), static_cast<int>((a >> 32) & 0xffff), bytes, 0x00020000};
    return d;
}
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void buffer_load4_to_lds(const int4_ext &descriptor, uint32_t ldsAddr, int laneBytes)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
                 :
                 : "s"(ldsAddr), "v"(laneBytes), "s"(descriptor)
                 : "memory", "m0");
}
#pragma clang diagnostic pop

// The rows of W as the wavefronts of dense_rows_split_kernel keep them: for wavefront q of the launch (outputs
// 32 q .. 32 q + 31), half j, chunk kc and lane (c = lane % 16, h = lane / 16), the three parts of
// W[32 q + 16 j + c][the inputs at positions 32 kc + 8h .. + 7] as 16 bytes each; position 16 G + 2 a + b of a chunk
// row holds input 16 G + 8 b + a (see the kernel).  parts[((q * 2 + j) * KC + kc) * 3 + part][lane].
__global__ __launch_bounds__(256) void dense_rows_split_weights_kernel(uint4_ext *parts, const float *w, int O, int K,
                                                                       int64_t wRow, int64_t wCol, int KC, int total)
{
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= total) return;
    const int lane = i & 63, c = lane & 15, h = lane >> 4;
    const int unit = i >> 6;   // (q * 2 + j) * KC + kc
    const int kc = unit % KC, qj = unit / KC;
    const int o = 16 * qj + c;
    float f[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const int pos = 32 * kc + 8 * h + e;
        const int k = (pos & ~15) + 8 * (pos & 1) + ((pos & 15) >> 1);
        f[e] = (o < O && k < K) ? w[o * wRow + k * wCol] : 0.0f;
    }
    const SplitPlanes s = split_bf16(f);
    uint4_ext *dst = parts + static_cast<size_t>(unit) * 3 * 64 + lane;
    dst[0] = s.hi;
    dst[64] = s.mid;
    dst[128] = s.lo;
}

template <int KC>
__global__ __launch_bounds__(64 * kDenseWaves) void dense_rows_split_kernel(DenseRowsArgs g)
{
    extern __shared__ __align__(16) char lds[];
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char *)lds));
    constexpr int ROW = 64 * KC + 16;                     // bytes per time sample of a plane
    constexpr int PLANE = kDenseTileT * ROW;              // bytes per plane
    constexpr int GROUPS = 4 * KC;                        // groups of 8 rows (1 KiB) of a raw tile
    constexpr int PAIRS = 2 * KC;                         // pairs of row groups = units of 64 lanes that are split
    constexpr int SR = (PAIRS + kDenseWaves - 1) / kDenseWaves;    // pairs per wavefront
    constexpr int RL = 2 * SR;                            // load instructions per wavefront and tile
    constexpr int RAW = RL * kDenseWaves * 1024;          // bytes per slot of the ring (whole instructions)
    static_assert(GROUPS <= RL * kDenseWaves, "a slot of the ring holds a tile");
    char *const ring = lds + 6 * PLANE;   // (behind the two sets of planes)
    uint32_t *flags = reinterpret_cast<uint32_t *>(ring + kDenseRing * RAW);   // [2][kDenseWaves]: a part beyond hi is not zero

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, h = lane >> 4;
    const int o0 = (blockIdx.y * kDenseWaves + wave) * 32;
    const bool working = o0 < g.O;   // (a layer with fewer outputs: the other wavefronts only help staging)
    // a work-group takes a contiguous range of tiles: consecutive tiles are the next 128 bytes of the same rows
    const uint32_t per = (g.tiles + gridDim.x - 1) / gridDim.x;
    uint32_t tile = blockIdx.x * per;
    const uint32_t end = min(g.tiles, tile + per);
    if (tile >= end) return;

    // this wavefront's rows of W, split: bw[j][kc] = W[o0 + 16 j + c][the inputs at positions 32 kc + 8h .. + 7]
    SplitPlanes bw[2][KC];
    {
        const uint4_ext *mine = g.wParts + static_cast<size_t>(blockIdx.y * kDenseWaves + wave) * (2 * KC * 3 * 64) + lane;
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int kc = 0; kc < KC; ++kc) {
                bw[j][kc].hi = mine[((j * KC + kc) * 3 + 0) * 64];
                bw[j][kc].mid = mine[((j * KC + kc) * 3 + 1) * 64];
                bw[j][kc].lo = mine[((j * KC + kc) * 3 + 2) * 64];
            }
    }

    // memory -> ring: an instruction moves a group of 8 rows, lane l the 16 bytes of row l / 8, samples 4 (l % 8) .. + 3.
    // A wavefront fetches the pairs of groups that it splits itself (pair wave + 8 r: groups 2 (wave + 8 r) and the
    // next), so its part of the ring is its own business; always RL instructions (what lies outside the tile arrives
    // as zeros)
    auto fetch = [&](uint32_t tile, int turn) {   // turn: which of the work-group's tiles this is (its slot: turn % 3)
        const bool live = tile < end;
        const int n = live ? static_cast<int>(tile / static_cast<uint32_t>(g.tilesPerItem)) : 0;
        const int t0 = (static_cast<int>(tile) - n * g.tilesPerItem) * kDenseTileT;
        const int4_ext bx = make_descriptor(g.x + n * g.xItem, live ? g.K * g.T * 4 : 0);
        const uint32_t slot = ldsBase + 6 * PLANE + (turn % kDenseRing) * RAW;
#pragma unroll
        for (int r = 0; r < RL; ++r) {
            const int grp = 2 * (wave + kDenseWaves * (r >> 1)) + (r & 1);
            const int k = 8 * grp + (lane >> 3), t = t0 + 4 * (lane & 7);
            buffer_load4_to_lds(bx, __builtin_amdgcn_readfirstlane(slot + grp * 1024),
                                masked_offset(k < g.K && t < g.T, (k * g.T + t) * 4));
        }
        __builtin_amdgcn_sched_barrier(0);   // (these stay where they are among the other memory instructions)
    };
    // ring -> planes: unit (pair of row groups 2 G, 2 G + 1; lane l): inputs 16 G + l / 8 and + 8, samples 4 (l % 8) .. + 3
    auto stage = [&](int turn) {
        const char *slot = ring + (turn % kDenseRing) * RAW;
        bool beyond = false;
#pragma unroll
        for (int r = 0; r < SR; ++r) {
            const int G = wave + kDenseWaves * r;
            if (G < PAIRS) {
                const float4 va = *reinterpret_cast<const float4 *>(slot + (2 * G) * 1024 + lane * 16);
                const float4 vb = *reinterpret_cast<const float4 *>(slot + (2 * G + 1) * 1024 + lane * 16);
                const float v[8] = {va.x, vb.x, va.y, vb.y, va.z, vb.z, va.w, vb.w};
                const SplitPlanes s = split_bf16(v);   // word e of a plane: the two inputs of sample 4 (l % 8) + e
                char *dst = lds + (turn & 1) * 3 * PLANE + (4 * (lane & 7)) * ROW + 32 * G + 4 * (lane >> 3);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    *reinterpret_cast<uint32_t *>(dst + e * ROW) = s.hi[e];
                    *reinterpret_cast<uint32_t *>(dst + PLANE + e * ROW) = s.mid[e];
                    *reinterpret_cast<uint32_t *>(dst + 2 * PLANE + e * ROW) = s.lo[e];
                    beyond |= (s.mid[e] | s.lo[e]) != 0u;
                }
            }
        }
        const bool any = __builtin_amdgcn_ballot_w64(beyond) != 0;
        if (lane == 0) flags[(turn & 1) * kDenseWaves + wave] = any ? 1u : 0u;
    };

    // One trip: the loads of the tile after the next go out (into the slot of the ring that this tile left in the
    // trip before), the next tile is split into the other set of planes, this tile is multiplied - in any order the
    // instructions like, the two do not depend on each other - and one barrier ends the trip.  The wait for the next
    // tile's loads leaves in flight what was issued after them: this trip's loads and the stores of the tile before
    // (4 per working wavefront; stores that the range check drops stand in for them before the first tile).  (Adding
    // to out: its loads come on top and the compiler waits for them; the wait here then only leaves this trip's
    // loads in flight.)
    const BufferRsrc none = make_buffer(g.out, 0);
    fetch(tile, 0);
    wait_vmem<0>();
    __syncthreads();
    stage(0);
    fetch(tile + 1, 1);
    if (working && !g.accumulate)
        for (int i = 0; i < 4; ++i) buffer_store4<kCached>(none, lane * 16, i * 1024, make_float4(0.0f, 0.0f, 0.0f, 0.0f));
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    for (int turn = 0;; ++turn) {
        fetch(tile + 2, turn + 2);
        if (working && !g.accumulate) wait_vmem<RL + 4>();
        else wait_vmem<RL>();
        stage(turn + 1);   // (the rows this wavefront fetched itself)
        // (the two wavefronts of a SIMD taking the trip's two jobs in opposite order, so that the matrix work of one
        // meets the splitting of the other, changed nothing: 67 us against 63 us on spikes, 104 against 107 on a
        // dense input)
        if (working) {
            const int n = static_cast<int>(tile / static_cast<uint32_t>(g.tilesPerItem));
            const int t0 = (static_cast<int>(tile) - n * g.tilesPerItem) * kDenseTileT;
            const BufferRsrc bo = make_buffer(g.out + static_cast<int64_t>(n) * g.O * g.T, g.O * g.T * 4);
            const bool allParts = __builtin_amdgcn_ballot_w64(lane < kDenseWaves && flags[(turn & 1) * kDenseWaves + (lane & 7)] != 0u) != 0;
            const char *base = lds + (turn & 1) * 3 * PLANE + c * ROW + 16 * h;
            // one sum per tile of 16 x 16 (two halves of the tile's samples tt x two halves of the wavefront's outputs
            // j), the smaller products of a chunk first.  The operands of a chunk of inputs are read while the chunk
            // before is multiplied.
            f32x4 acc[2][2];
#pragma unroll
            for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[tt][j] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
            if (allParts) {
                // (one half of the samples at a time: three planes of two halves, twice, would not fit the registers)
                uint4_ext xh[2], xm[2], xl[2];
                auto read = [&](int set, int step) {
                    const char *row = base + 16 * (step & 1) * ROW + 64 * (step >> 1);
                    xh[set] = *reinterpret_cast<const uint4_ext *>(row);
                    xm[set] = *reinterpret_cast<const uint4_ext *>(row + PLANE);
                    xl[set] = *reinterpret_cast<const uint4_ext *>(row + 2 * PLANE);
                };
                read(0, 0);
#pragma unroll
                for (int step = 0; step < 2 * KC; ++step) {
                    const int set = step & 1, tt = step & 1, kc = step >> 1;
                    if (step + 1 < 2 * KC) read(set ^ 1, step + 1);
                    __builtin_amdgcn_sched_barrier(0);   // (issued here, ahead of the matrix instructions of this step)
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[tt][j] = mfma_bf16(xh[set], bw[j][kc].lo, acc[tt][j]);
                        acc[tt][j] = mfma_bf16(xl[set], bw[j][kc].hi, acc[tt][j]);
                        acc[tt][j] = mfma_bf16(xm[set], bw[j][kc].mid, acc[tt][j]);
                        acc[tt][j] = mfma_bf16(xh[set], bw[j][kc].mid, acc[tt][j]);
                        acc[tt][j] = mfma_bf16(xm[set], bw[j][kc].hi, acc[tt][j]);
                        acc[tt][j] = mfma_bf16(xh[set], bw[j][kc].hi, acc[tt][j]);
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            } else {
                uint4_ext xh[2][2];
                auto read = [&](int set, int kc) {
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt) xh[set][tt] = *reinterpret_cast<const uint4_ext *>(base + 16 * tt * ROW + 64 * kc);
                };
                read(0, 0);
#pragma unroll
                for (int kc = 0; kc < KC; ++kc) {
                    const int set = kc & 1;
                    if (kc + 1 < KC) read(set ^ 1, kc + 1);
                    __builtin_amdgcn_sched_barrier(0);   // (issued here, ahead of the matrix instructions of this step)
#pragma unroll
                    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            acc[tt][j] = mfma_bf16(xh[set][tt], bw[j][kc].lo, acc[tt][j]);
                            acc[tt][j] = mfma_bf16(xh[set][tt], bw[j][kc].mid, acc[tt][j]);
                            acc[tt][j] = mfma_bf16(xh[set][tt], bw[j][kc].hi, acc[tt][j]);
                        }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) {
                const int t = t0 + 16 * tt + 4 * h;
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    const int o = o0 + 16 * j + c;
                    const int off = masked_offset(o < g.O && t < g.T, (o * g.T + t) * 4);
                    float4 y = make_float4(acc[tt][j][0], acc[tt][j][1], acc[tt][j][2], acc[tt][j][3]);
                    if (g.accumulate) {
                        const float4 old = buffer_load4<kCached>(bo, off, 0);
                        y = make_float4(y.x + old.x, y.y + old.y, y.z + old.z, y.w + old.w);
                    }
                    // (a store covers 64 bytes of each of 16 output rows, and the tile's other half completes the
                    // lines: cached, so that L2 puts them together)
                    buffer_store4<kCached>(bo, off, 0, y);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (++tile >= end) break;
        __syncthreads();
    }
}

static size_t dense_rows_lds(int kc)
{
    const int rl = 2 * ((2 * kc + kDenseWaves - 1) / kDenseWaves);
    return static_cast<size_t>(6) * kDenseTileT * (64 * kc + 16) + static_cast<size_t>(kDenseRing) * rl * kDenseWaves * 1024 +
           2 * kDenseWaves * 4;
}

template <int KC>
static void launch_dense_rows(const DenseRowsArgs &g, dim3 grid, hipStream_t st)
{
    hipLaunchKernelGGL((dense_rows_split_kernel<KC>), grid, dim3(64 * kDenseWaves), dense_rows_lds(KC), st, g);
}

}  // namespace slayer

// bytes of the split weights of one launch: wavefronts x halves x chunks x parts x 1 KiB
static int64_t dense_rows_parts_bytes(int64_t O, int kc)
{
    const int64_t wavefronts = (O + 32 * slayer::kDenseWaves - 1) / (32 * slayer::kDenseWaves) * slayer::kDenseWaves;
    return wavefronts * 2 * kc * 3 * 1024;
}

extern "C" int slayer_dense_rows_supported(int64_t N, int64_t K, int64_t O, int64_t T)
{
    const int64_t lim = (1LL << 31) - 64;
    return N >= 1 && K >= 1 && O >= 1 && T >= 4 && T % 4 == 0 && K * T * 4 < lim && O * T * 4 < lim &&
           N * ((T + slayer::kDenseTileT - 1) / slayer::kDenseTileT) < (1LL << 31) && O <= 65535 * 256 && K * O * 4 < lim;
}

extern "C" int64_t slayer_dense_rows_workspace_bytes(int64_t K, int64_t O)
{
    if (K < 1 || O < 1) return 0;
    return dense_rows_parts_bytes(O, static_cast<int>((K + 31) / 32));   // (blocks of whole chunks: the chunks add up)
}

extern "C" int slayer_dense_rows_f32(float *out, const float *w, const float *x, void *workspace, int64_t N, int64_t K,
                                     int64_t O, int64_t T, int64_t wRow, int64_t wCol, void *stream)
{
    using namespace slayer;
    if (N < 0 || K < 0 || O < 0 || T < 0) return SLAYER_EINVAL;
    if (N == 0 || O == 0 || T == 0) return SLAYER_OK;
    if (!out || (K > 0 && (!w || !x || !workspace))) return SLAYER_EINVAL;
    if (K == 0 || !slayer_dense_rows_supported(N, K, O, T) || !aligned16(out) || !aligned16(x) || !aligned16(workspace))
        return SLAYER_EUNSUPPORTED;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int tilesPerItem = static_cast<int>((T + kDenseTileT - 1) / kDenseTileT);
    const int64_t tiles = N * tilesPerItem;
    const dim3 grid(static_cast<unsigned>(tiles < compute_units() ? tiles : compute_units()),
                    static_cast<unsigned>((O + 32 * kDenseWaves - 1) / (32 * kDenseWaves)));
    // inputs beyond what a launch takes: blocks of them, one launch each, adding up in out
    constexpr int kBlock = 32 * kDenseMaxChunks;
    const int64_t blocks = (K + kBlock - 1) / kBlock;
    const int64_t per = (((K + blocks - 1) / blocks) + 31) / 32 * 32;   // equal blocks of whole chunks
    char *parts = static_cast<char *>(workspace);
    for (int64_t k0 = 0, i = 0; k0 < K; k0 += per, ++i) {
        const int kk = static_cast<int>(K - k0 < per ? K - k0 : per);
        const int kc = (kk + 31) / 32;
        const int total = static_cast<int>(dense_rows_parts_bytes(O, kc) / (3 * 16));
        hipLaunchKernelGGL(dense_rows_split_weights_kernel, dim3((total + 255) / 256), dim3(256), 0, st,
                           reinterpret_cast<uint4_ext *>(parts), w + k0 * wCol, static_cast<int>(O), kk, wRow, wCol, kc, total);
        DenseRowsArgs g{out, x + k0 * T, reinterpret_cast<const uint4_ext *>(parts), static_cast<int>(N), static_cast<int>(O), kk,
                        static_cast<int>(T), K * T, i > 0 ? 1 : 0, tilesPerItem, static_cast<uint32_t>(tiles)};
        switch (kc) {
            case 1: launch_dense_rows<1>(g, grid, st); break;
            case 2: launch_dense_rows<2>(g, grid, st); break;
            case 3: launch_dense_rows<3>(g, grid, st); break;
            case 4: launch_dense_rows<4>(g, grid, st); break;
            case 5: launch_dense_rows<5>(g, grid, st); break;
            case 6: launch_dense_rows<6>(g, grid, st); break;
            default: launch_dense_rows<7>(g, grid, st); break;
        }
        parts += dense_rows_parts_bytes(O, kc);
    }
    return launch_status();
}

// ---- the weight gradient of the same layers -------------------------------------------------------------------------
//
//     gradW[o][k] = sum_{n, t} gradOut[n][o][t] * x[n][k][t]
//
// Both operands have the reduction axis, time, innermost: a lane's operand of v_mfma_f32_16x16x32_bf16 - 8 consecutive
// samples of one row - is 32 contiguous bytes of either tensor.  A work-group of 8 wavefronts owns ALL outputs and up
// to 208 inputs (16 x 13 tiles of 16 x 16, wavefront w the tiles of output rows 32 w .. 32 w + 31: at most 104
// accumulator registers; layers with more inputs take a launch per block of inputs) and a contiguous range of chunks
// of 32 samples.  Per chunk the rows of x travel into a ring in LDS and are split into three planes [k][t] of bf16
// there, once, for all wavefronts (pitch 80 bytes: the 16 rows of an operand read spread over the banks); a
// wavefront's own 32 rows of gradOut come straight from memory into registers, one chunk ahead, and are split there.
// Spike tiles of x take three of the six products, as in the kernel above.  Every work-group writes its sums to a row
// of `partial`; a second kernel adds the
// rows in a fixed order.
namespace slayer {

// floats between the work-groups' sums in the workspace: a multiple of four, for the sum kernel's 16-byte loads
__host__ __device__ inline int64_t dense_wgrad_pitch(int64_t O, int64_t K) { return (O * K + 3) / 4 * 4; }

constexpr int kWgradMaxInputs = 208;   // per launch: 13 tiles of 16, what the planes of a chunk leave room for in LDS
constexpr int kWgradPitch = 80;   // bytes per input row of a plane: 32 samples of bf16 and 16 bytes of padding

struct DenseWgradArgs {
    float *partial;
    const float *gradOut, *x;
    int N, O, K, T;
    int k0, kEnd;            // the inputs this launch covers
    int chunksPerItem;
    uint32_t chunks;
};

template <int KT>   // tiles of 16 inputs
__global__ __launch_bounds__(64 * kDenseWaves) void dense_wgrad_split_kernel(DenseWgradArgs g)
{
    extern __shared__ __align__(16) char lds[];
    constexpr int PLANE = 16 * KT * kWgradPitch;            // bytes per plane
    constexpr int GROUPS = 2 * KT;                          // groups of 8 rows (1 KiB) of a raw tile
    constexpr int RL = (GROUPS + kDenseWaves - 1) / kDenseWaves;   // groups, i.e. load instructions, per wavefront
    constexpr int RAW = GROUPS * 1024;
    const uint32_t ldsBase = static_cast<uint32_t>(reinterpret_cast<size_t>((__attribute__((address_space(3))) char *)lds));
    char *const ring = lds + 6 * PLANE;
    uint32_t *flags = reinterpret_cast<uint32_t *>(ring + 2 * RAW);   // [2][kDenseWaves]

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, c = lane & 15, h = lane >> 4;
    const int o0 = (blockIdx.y * kDenseWaves + wave) * 32;
    const bool working = o0 < g.O;
    const uint32_t per = (g.chunks + gridDim.x - 1) / gridDim.x;
    uint32_t chunk = blockIdx.x * per;
    const uint32_t end = min(g.chunks, chunk + per);

    f32x4 acc[2][KT];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) acc[j][kt] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};

    auto place = [&](uint32_t ch, int &n, int &t0) {
        n = static_cast<int>(ch / static_cast<uint32_t>(g.chunksPerItem));
        t0 = (static_cast<int>(ch) - n * g.chunksPerItem) * 32;
    };
    // x: memory -> ring (group wave + 8 r: rows 8 (wave + 8 r) .. + 7; lane l: row l / 8, samples 4 (l % 8) .. + 3)
    auto fetch = [&](uint32_t ch, int turn) {
        const bool live = ch < end;
        int n, t0;
        place(live ? ch : 0, n, t0);
        const int4_ext bx = make_descriptor(g.x + static_cast<int64_t>(n) * g.K * g.T, live ? g.K * g.T * 4 : 0);
        const uint32_t slot = ldsBase + 6 * PLANE + (turn & 1) * RAW;
#pragma unroll
        for (int r = 0; r < RL; ++r) {
            const int grp = wave + kDenseWaves * r;
            if (grp >= GROUPS) break;
            const int k = g.k0 + 8 * grp + (lane >> 3), t = t0 + 4 * (lane & 7);
            buffer_load4_to_lds(bx, __builtin_amdgcn_readfirstlane(slot + grp * 1024),
                                masked_offset(k < g.kEnd && t < g.T, (k * g.T + t) * 4));
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // ring -> planes (the groups this wavefront fetched itself, two at a time)
    auto stage = [&](int turn) {
        const char *slot = ring + (turn & 1) * RAW;
        char *planes = lds + (turn & 1) * 3 * PLANE;
        bool beyond = false;
#pragma unroll
        for (int r = 0; r < RL; r += 2) {
            const int ga = wave + kDenseWaves * r, gb = wave + kDenseWaves * (r + 1);
            if (ga < GROUPS) {
                const float4 va = *reinterpret_cast<const float4 *>(slot + ga * 1024 + lane * 16);
                const float4 vb = (r + 1 < RL && gb < GROUPS) ? *reinterpret_cast<const float4 *>(slot + gb * 1024 + lane * 16)
                                                              : make_float4(0.0f, 0.0f, 0.0f, 0.0f);
                const float v[8] = {va.x, va.y, va.z, va.w, vb.x, vb.y, vb.z, vb.w};
                const SplitPlanes s = split_bf16(v);   // words 0, 1: the four samples of row a; words 2, 3: of row b
                char *da = planes + (8 * ga + (lane >> 3)) * kWgradPitch + 8 * (lane & 7);
                *reinterpret_cast<uint2 *>(da) = make_uint2(s.hi[0], s.hi[1]);
                *reinterpret_cast<uint2 *>(da + PLANE) = make_uint2(s.mid[0], s.mid[1]);
                *reinterpret_cast<uint2 *>(da + 2 * PLANE) = make_uint2(s.lo[0], s.lo[1]);
                if (r + 1 < RL && gb < GROUPS) {
                    char *db = planes + (8 * gb + (lane >> 3)) * kWgradPitch + 8 * (lane & 7);
                    *reinterpret_cast<uint2 *>(db) = make_uint2(s.hi[2], s.hi[3]);
                    *reinterpret_cast<uint2 *>(db + PLANE) = make_uint2(s.mid[2], s.mid[3]);
                    *reinterpret_cast<uint2 *>(db + 2 * PLANE) = make_uint2(s.lo[2], s.lo[3]);
                }
                beyond |= ((s.mid[0] | s.mid[1]) | (s.mid[2] | s.mid[3]) | (s.lo[0] | s.lo[1]) | (s.lo[2] | s.lo[3])) != 0u;
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        const bool any = __builtin_amdgcn_ballot_w64(beyond) != 0;
        if (lane == 0) flags[(turn & 1) * kDenseWaves + wave] = any ? 1u : 0u;
    };
    // gradOut: this lane's samples 8h .. 8h + 7 of rows o0 + 16 j + c of a chunk, straight into registers
    float4 ga[2][2];
    auto fetch_grad = [&](uint32_t ch) {
        const bool live = ch < end;
        int n, t0;
        place(live ? ch : 0, n, t0);
        const BufferRsrc bg = make_buffer(g.gradOut + static_cast<int64_t>(n) * g.O * g.T, live ? g.O * g.T * 4 : 0);
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int o = o0 + 16 * j + c, t = t0 + 8 * h;
            ga[j][0] = buffer_load4<kCached>(bg, masked_offset(o < g.O && t < g.T, (o * g.T + t) * 4), 0);
            ga[j][1] = buffer_load4<kCached>(bg, masked_offset(o < g.O && t + 4 < g.T, (o * g.T + t + 4) * 4), 0);
        }
    };

    if (chunk < end) {
        fetch_grad(chunk);
        fetch(chunk, 0);
        wait_vmem<0>();
        stage(0);
        __syncthreads();
        for (int turn = 0;; ++turn) {
            // this chunk's rows of gradOut, split (they were fetched a trip ago); then the next chunk's go out, and
            // the rows of x of the chunk after the next
            SplitPlanes a[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const float v[8] = {ga[j][0].x, ga[j][0].y, ga[j][0].z, ga[j][0].w, ga[j][1].x, ga[j][1].y, ga[j][1].z, ga[j][1].w};
                a[j] = split_bf16(v);
                __builtin_amdgcn_sched_barrier(0);
            }
            fetch_grad(chunk + 1);
            __builtin_amdgcn_sched_barrier(0);
            if (turn == 0) {
                fetch(chunk + 1, 1);
                wait_vmem<0>();      // (the first trip has nothing in flight to hide this behind)
            } else {
                // the next chunk's rows of x were fetched a trip ago; behind them: this trip's four loads of gradOut
                wait_vmem<4>();
            }
            stage(turn + 1);
            fetch(chunk + 2, turn + 2);   // (into the slot whose rows, this chunk's, were split a trip ago)
            if (working) {
                const bool allParts = __builtin_amdgcn_ballot_w64(lane < kDenseWaves && flags[(turn & 1) * kDenseWaves + (lane & 7)] != 0u) != 0;
                const char *base = lds + (turn & 1) * 3 * PLANE + c * kWgradPitch + 16 * h;
                // (one loop with the test inside: as two loops under the test, the compiler kept the operands of both
                // in registers at once)
#pragma unroll
                for (int kt = 0; kt < KT; ++kt) {
                    if (allParts) {
                        const uint4_ext xm = *reinterpret_cast<const uint4_ext *>(base + PLANE + 16 * kt * kWgradPitch);
                        const uint4_ext xl = *reinterpret_cast<const uint4_ext *>(base + 2 * PLANE + 16 * kt * kWgradPitch);
#pragma unroll
                        for (int j = 0; j < 2; ++j) {
                            acc[j][kt] = mfma_bf16(a[j].hi, xl, acc[j][kt]);
                            acc[j][kt] = mfma_bf16(a[j].mid, xm, acc[j][kt]);
                            acc[j][kt] = mfma_bf16(a[j].hi, xm, acc[j][kt]);
                        }
                    }
                    const uint4_ext xh = *reinterpret_cast<const uint4_ext *>(base + 16 * kt * kWgradPitch);
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        acc[j][kt] = mfma_bf16(a[j].lo, xh, acc[j][kt]);
                        acc[j][kt] = mfma_bf16(a[j].mid, xh, acc[j][kt]);
                        acc[j][kt] = mfma_bf16(a[j].hi, xh, acc[j][kt]);
                    }
                }
            }
            __builtin_amdgcn_sched_barrier(0);
            if (++chunk >= end) break;
            __syncthreads();
        }
    }
    // this work-group's sums: lane (c, h) holds rows 4h .. 4h + 3, column c of every tile
    if (working) {
        float *row = g.partial + static_cast<int64_t>(blockIdx.x) * dense_wgrad_pitch(g.O, g.K);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const int k = g.k0 + 16 * kt + c;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int o = o0 + 16 * j + 4 * h + r;
                    if (o < g.O && k < g.kEnd) row[o * g.K + k] = acc[j][kt][r];
                }
            }
    }
}

// out[i] = sum of the rows of partial, in a fixed order: 16 threads share a column of four sums, each adds every
// sixteenth row, and one of them adds the sixteen results (rows lie `pitch` floats apart, a multiple of 4 that holds
// n; rows == 0 writes zeros)
__global__ __launch_bounds__(256) void dense_wgrad_sum_kernel(float *out, const float *partial, int rows, int n, int64_t pitch)
{
    __shared__ float4 part[16][17];
    const int col = threadIdx.x & 15, slice = threadIdx.x >> 4;
    const int i = (blockIdx.x * 16 + col) * 4;
    float4 s = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
    if (i < n) {
        const float *p = partial + i;
        int r = slice;
        for (; r + 48 < rows; r += 64) {
            const float4 a = *reinterpret_cast<const float4 *>(p + r * pitch);
            const float4 b = *reinterpret_cast<const float4 *>(p + (r + 16) * pitch);
            const float4 c = *reinterpret_cast<const float4 *>(p + (r + 32) * pitch);
            const float4 d = *reinterpret_cast<const float4 *>(p + (r + 48) * pitch);
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
            s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
            s.x += c.x; s.y += c.y; s.z += c.z; s.w += c.w;
            s.x += d.x; s.y += d.y; s.z += d.z; s.w += d.w;
        }
        for (; r < rows; r += 16) {
            const float4 a = *reinterpret_cast<const float4 *>(p + r * pitch);
            s.x += a.x; s.y += a.y; s.z += a.z; s.w += a.w;
        }
    }
    part[slice][col] = s;
    __syncthreads();
    if (slice == 0 && i < n) {
        float4 t = part[0][col];
        for (int q = 1; q < 16; ++q) {
            const float4 a = part[q][col];
            t.x += a.x; t.y += a.y; t.z += a.z; t.w += a.w;
        }
        if (i + 3 < n) {
            out[i] = t.x; out[i + 1] = t.y; out[i + 2] = t.z; out[i + 3] = t.w;   // (out need not be 16-byte aligned)
        } else {
            out[i] = t.x;
            if (i + 1 < n) out[i + 1] = t.y;
            if (i + 2 < n) out[i + 2] = t.z;
        }
    }
}

template <int KT>
static void launch_dense_wgrad(const DenseWgradArgs &g, dim3 grid, hipStream_t st)
{
    const size_t lds = static_cast<size_t>(6) * 16 * KT * kWgradPitch + static_cast<size_t>(2) * 2 * KT * 1024 + 2 * kDenseWaves * 4;
    hipLaunchKernelGGL((dense_wgrad_split_kernel<KT>), grid, dim3(64 * kDenseWaves), lds, st, g);
}

static int dense_wgrad_groups(int64_t N, int64_t T)
{
    const int64_t chunks = N * ((T + 31) / 32);
    return static_cast<int>(chunks < compute_units() ? chunks : compute_units());
}

}  // namespace slayer

extern "C" int slayer_dense_rows_grad_weight_supported(int64_t N, int64_t K, int64_t O, int64_t T)
{
    const int64_t lim = (1LL << 31) - 64;
    return N >= 1 && K >= 1 && K <= 448 && O >= 1 && O <= 256 && T >= 4 && T % 4 == 0 && K * T * 4 < lim && O * T * 4 < lim &&
           N * ((T + 31) / 32) < (1LL << 31);
}

extern "C" int64_t slayer_dense_rows_grad_weight_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T)
{
    if (N < 1 || K < 1 || O < 1 || T < 1) return 0;
    return static_cast<int64_t>(slayer::dense_wgrad_groups(N, T)) * slayer::dense_wgrad_pitch(O, K) * 4;
}

extern "C" int slayer_dense_rows_grad_weight_f32(float *gradW, const float *gradOut, const float *x, void *workspace, int64_t N,
                                                 int64_t K, int64_t O, int64_t T, void *stream)
{
    using namespace slayer;
    if (N < 0 || K < 0 || O < 0 || T < 0) return SLAYER_EINVAL;
    if (K == 0 || O == 0) return SLAYER_OK;
    if (!gradW) return SLAYER_EINVAL;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (N == 0 || T == 0) {
        const int n = static_cast<int>(O * K);   // (a sum over no rows: zeros, from a kernel a caller may capture)
        hipLaunchKernelGGL(dense_wgrad_sum_kernel, dim3((n + 63) / 64), dim3(256), 0, st, gradW, static_cast<const float *>(nullptr), 0, n, dense_wgrad_pitch(O, K));
        return launch_status();
    }
    if (!gradOut || !x || !workspace) return SLAYER_EINVAL;
    if (!slayer_dense_rows_grad_weight_supported(N, K, O, T) || !aligned16(gradOut) || !aligned16(x) || !aligned16(workspace))
        return SLAYER_EUNSUPPORTED;
    const int chunksPerItem = static_cast<int>((T + 31) / 32);
    const int64_t chunks = N * chunksPerItem;
    const int groups = dense_wgrad_groups(N, T);
    // up to 208 inputs a launch; more go in even blocks
    const int blocks = static_cast<int>((K + kWgradMaxInputs - 1) / kWgradMaxInputs);
    const int per = static_cast<int>(((K + blocks - 1) / blocks + 15) / 16 * 16);
    const dim3 grid(static_cast<unsigned>(groups), 1);
    for (int k0 = 0; k0 < K; k0 += per) {
        const int kEnd = static_cast<int>(K < k0 + per ? K : k0 + per);
        DenseWgradArgs g{static_cast<float *>(workspace), gradOut, x, static_cast<int>(N), static_cast<int>(O), static_cast<int>(K),
                         static_cast<int>(T), k0, kEnd, chunksPerItem, static_cast<uint32_t>(chunks)};
        switch ((kEnd - k0 + 15) / 16) {
#define SLAYER_DENSE_WGRAD(KT) case KT: launch_dense_wgrad<KT>(g, grid, st); break
            SLAYER_DENSE_WGRAD(1); SLAYER_DENSE_WGRAD(2); SLAYER_DENSE_WGRAD(3); SLAYER_DENSE_WGRAD(4); SLAYER_DENSE_WGRAD(5);
            SLAYER_DENSE_WGRAD(6); SLAYER_DENSE_WGRAD(7); SLAYER_DENSE_WGRAD(8); SLAYER_DENSE_WGRAD(9); SLAYER_DENSE_WGRAD(10);
            SLAYER_DENSE_WGRAD(11); SLAYER_DENSE_WGRAD(12);
            default: launch_dense_wgrad<13>(g, grid, st); break;
#undef SLAYER_DENSE_WGRAD
        }
    }
    const int n = static_cast<int>(O * K);
    hipLaunchKernelGGL(dense_wgrad_sum_kernel, dim3((n + 63) / 64), dim3(256), 0, st, gradW, static_cast<const float *>(workspace),
                       groups, n, dense_wgrad_pitch(O, K));
    return launch_status();
}

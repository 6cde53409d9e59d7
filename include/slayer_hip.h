/*
 * slayer_hip.h - C ABI of libslayer_hip.so: SLAYER's per-neuron temporal kernels for AMD
 * MI355X (gfx950), hand-written HIP.
 *
 * This is the drop-in boundary for the reference's two pybind11 extension modules,
 * `slayerCuda` (src/cuda/slayerKernels.cu:136-145) and `slayerLoihiCuda`
 * (src/cuda/slayerLoihiKernels.cu:48-51).  Each entry point below names the reference
 * binding it replaces.
 *
 * Conventions shared by every entry point
 *   - All tensors are dense, contiguous float32 device buffers shaped [nNeurons][T] with time
 *     innermost ("neuron row" = T consecutive samples).  Any leading tensor shape
 *     (N,C,H,W,...) is flattened into nNeurons by the caller.
 *   - Pointers are device pointers valid on the CURRENT HIP device; the caller selects the
 *     device (the reference bindings call cudaSetDevice on the tensor's device).
 *   - `stream` is a hipStream_t passed as void* (NULL = the default stream).  Calls only
 *     enqueue work: no allocation, no free, no host synchronisation, and no state kept between
 *     calls - with two exceptions, both stated where they are declared: the process-wide test knob
 *     slayer_force_generic_kernels, and the fixed device array of slayer_delay_grad_static_f32.
 *   - The library never allocates device memory.  Outputs (and the workspaces of
 *     slayer_delay_grad_f32, slayer_synapse_conv_grad_weight_f32, slayer_dense_events_f32,
 *     slayer_dense_events_grad_weight_f32 and slayer_spike_loss_f32) are allocated by
 *     the caller.
 *   - Return value: SLAYER_OK (0) or one of the SLAYER_E* codes; nothing has been launched
 *     when a SLAYER_EINVAL / SLAYER_EUNSUPPORTED code is returned.  Empty tensors
 *     (nNeurons == 0 or T == 0) are a successful no-op.
 */
#ifndef SLAYER_HIP_H_INCLUDED
#define SLAYER_HIP_H_INCLUDED

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define SLAYER_HIP_ABI_VERSION 1

enum {
    SLAYER_OK = 0,
    SLAYER_EINVAL = 1,       /* null pointer, negative size, refDelay == 0, ... */
    SLAYER_EUNSUPPORTED = 2, /* size outside what the kernels index (see each function) */
    SLAYER_ELAUNCH = 3       /* the HIP runtime reported an error for the launch */
};

/* ABI version of the loaded library (== SLAYER_HIP_ABI_VERSION it was built with). */
int slayer_hip_abi_version(void);

/* Static, human readable text for a status code. */
const char *slayer_status_string(int status);

/* Text of the last HIP runtime error seen by this thread inside the library ("" if none). */
const char *slayer_last_hip_error(void);

/*
 * Debug/validation knob, process wide: 0 (default) = tiled LDS kernels wherever the sizes
 * allow; 1 = always use the generic one-thread-per-sample / one-thread-per-neuron kernels
 * (the ones that also serve sizes the tiled kernels do not cover).  Both produce the same
 * results.  Returns the previous value.  No counterpart in the reference.
 */
int slayer_force_generic_kernels(int on);

/*
 * SRM spike generation with refractory feedback.
 * Replaces slayerCuda.getSpikes -> getSpikesCuda (src/cuda/slayerKernels.cu:14-39),
 * kernel src/cuda/spikeKernels.h:9-38.
 *
 * For each neuron row, t ascending: if u[t] >= theta then s[t] = 1/Ts and
 * u[t+j] += nu[j] for j in [0, nuSize) with t+j < T; else s[t] = 0.  `u` is updated IN
 * PLACE (it holds the post-refractory membrane potential on return); `s` is written.
 * Results are bit-identical to the sequential fp32 loop.  nuSize may be 0.
 */
int slayer_get_spikes_f32(float *s, float *u, const float *nu, int64_t nNeurons, int64_t T,
                          int64_t nuSize, float theta, float Ts, void *stream);

/*
 * Causal temporal convolution (PSP filter, forward).
 * Replaces slayerCuda.conv -> convCuda (src/cuda/slayerKernels.cu:41-57),
 * kernel src/cuda/convKernels.h:10-35.
 *
 * out[n][t] = Ts * sum_{i=0..F-1, t-i>=0} in[n][t-i] * filt[i], accumulated in fp32 by
 * fused multiply-add in tap order i = 0,1,...  `out` must not alias `in`.  F >= 1... F == 0
 * yields zeros.
 *
 * Rows of whole 16-byte vectors with 34 to 129 taps: tiles of 16 rows whose input is dense (more than one
 * 16-byte vector in five holds a non-zero sample) are computed on the matrix cores, which add the terms in
 * another order than the sequential loop: those results agree with it to rounding (every output within
 * 1e-5 of the sum of the magnitudes of its own terms; measured about 1e-7 of the largest output).  Tiles of
 * spike trains (almost all zeros) and all other shapes match the fused-multiply-add loop bit for bit.
 */
int slayer_conv_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T,
                    int64_t F, float Ts, void *stream);

/*
 * Anti-causal temporal correlation (PSP filter, backward; adjoint of slayer_conv_f32).
 * Replaces slayerCuda.corr -> corrCuda (src/cuda/slayerKernels.cu:59-75),
 * kernel src/cuda/convKernels.h:37-62.
 *
 * out[n][t] = Ts * sum_{i=0..F-1, t+i<T} in[n][t+i] * filt[i].
 *
 * Rows of whole 16-byte vectors with 34 to 129 taps are computed on the matrix cores, which add the
 * terms in another order than the sequential loop - whole rows of up to 316 samples whose T / 4 is odd
 * (T = 300) with bf16 instructions over a three-way split of samples and taps, the others with fp32
 * instructions: those results agree with the loop to rounding (every output within 1e-6 of the sum of the
 * magnitudes of its own terms; parts of samples and taps below 2^-126 are read as zero, at most
 * 2^-124 * (sum |filt| + sum |in| over an output's window) in absolute terms), all others bit for bit
 * with the fused-multiply-add loop.
 */
int slayer_corr_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T,
                    int64_t F, float Ts, void *stream);

/*
 * Time shift by one delay for all rows, delay given by value.
 * Replaces slayerCuda.shift(Tensor, float[, Ts]) -> shiftFlCuda / shiftFl1Cuda
 * (src/cuda/slayerKernels.cu:114-134), kernel src/cuda/shiftKernels.h:9-34.
 *
 * k = (int)(delay / Ts)  (fp32 quotient truncated toward zero);
 * out[n][t] = (0 <= t-k < T) ? in[n][t-k] : 0.  `out` must not alias `in`.
 */
int slayer_shift_f32(float *out, const float *in, float delay, int64_t nNeurons, int64_t T,
                     float Ts, void *stream);

/*
 * Time shift with delays read from device memory.
 * Replaces slayerCuda.shift(Tensor, Tensor[, Ts]) -> shiftCuda / shift1Cuda
 * (src/cuda/slayerKernels.cu:77-112), kernels src/cuda/shiftKernels.h:9-61.
 *
 * lutSize == 1: every row is shifted by lut[0] (read on the device: unlike the reference's
 * `.item()` there is no host synchronisation).  Otherwise lutSize must equal nPerBatch and
 * row (b, m) of the [nBatch][nPerBatch][T] tensor is shifted by lut[m]; one launch covers
 * all batches.  `sign` (+1 or -1) multiplies every delay before use, so that the backward
 * pass (shift by -delay, src/slayer.py:957,979) needs no negated copy of the table.
 */
int slayer_shift_lut_f32(float *out, const float *in, const float *lut, int64_t lutSize,
                         int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts, float sign,
                         void *stream);

/*
 * Surrogate gradient of the spike function, fused into one pass.
 * Replaces the torch expression chain of _spikeFunction.backward (src/slayer.py:857-865) and
 * slayerLoihi._spike.backward (src/slayerLoihi.py:278-283); native precedent evalRhoKernel
 * (src/cuda/spikeKernels.h:41-52).
 *
 * gradIn[i] = gradOut[i] * (scale / tau) * exp(-|u[i] - theta| / tau), tau = tauRho * theta.
 * gradIn may alias gradOut.  tau must be non-zero.
 */
int slayer_spike_bwd_f32(float *gradIn, const float *gradOut, const float *u, float theta,
                         float tau, float scale, int64_t numel, void *stream);

/*
 * Backward pass of the Loihi neuron in one kernel: surrogate gradient, then correlation with
 * the PSP kernel.  Replaces the body of slayerLoihi._spike.backward (src/slayerLoihi.py:278-283:
 * the spikePdf expression chain followed by slayerCuda.corr, src/cuda/slayerKernels.cu:59-75).
 *
 * gradIn[n][t] = Ts * sum_{i<F} [t+i < T] w[n][t+i] * filt[i],
 * w[n][t]      = gradOut[n][t] * (scale / tau) * exp(-|u[n][t] - theta| / tau).
 * The values of slayer_spike_bwd_f32 followed by slayer_corr_f32, without the intermediate tensor: rows of
 * whole 16-byte vectors with 34 to 129 taps are summed on the matrix cores and agree with the sequential
 * fused-multiply-add loop to rounding (1e-5, as for slayer_corr_f32), all other shapes bit for bit.
 * gradIn must not alias the inputs.  tau must be non-zero.
 */
int slayer_spike_bwd_corr_f32(float *gradIn, const float *gradOut, const float *u,
                              const float *filt, int64_t nNeurons, int64_t T, int64_t F,
                              float theta, float tau, float scale, float Ts, void *stream);

/*
 * PSP filter followed by the spike function in one kernel, for layers that apply them back to
 * back: spike(psp(x)), the ordering of the reference's MLP example
 * (example/02_NMNIST_MLP/nmnistMLP.py:59-60).  Replaces the call pair slayerCuda.conv
 * (src/cuda/slayerKernels.cu:41-57) -> slayerCuda.getSpikes (src/cuda/slayerKernels.cu:14-39).
 *
 * u = Ts * conv(a, srm), then s and the refractory update of u as in slayer_get_spikes_f32, without
 * the round trip of u through memory when rows are whole 16-byte vectors of at most 352 samples,
 * nuSize <= 24 and F <= 160.  Filters of 34 to 113 taps (on rows of at least 16 samples) are summed on the
 * matrix cores (bf16 instructions over a three-way split of samples and taps, as in slayer_corr_f32; 114 to
 * 129 taps: slayer_conv_f32, then slayer_get_spikes_f32), which add the terms in another order than the
 * sequential fused-multiply-add loop: the
 * potentials agree with the reference's to rounding (1e-5 of the sum of each output's terms' magnitudes), the
 * spikes are the spike function of exactly these potentials, and a tile of 16 rows that holds a non-finite
 * sample is filtered with the sequential loop (the reference's bits, infinities and NaNs where it puts them).
 * All other filters run the sequential loop for every input (the reference's bits).  Other shapes run the
 * two kernels one after the other.  u and s must not alias a.
 */
int slayer_psp_spike_f32(float *s, float *u, const float *a, const float *srm, const float *nu,
                         int64_t nNeurons, int64_t T, int64_t F, int64_t nuSize, float theta,
                         float Ts, void *stream);

/*
 * PSP filtering with an alpha kernel, filt[k] = mult * (k Ts / tau) * exp(1 - k Ts / tau) for k < F - the SRM
 * kernel that the reference's layers build (src/slayer.py:98-123) and hand to slayerCuda.conv / corr
 * (src/slayer.py:878-899, src/cuda/slayerKernels.cu:41-75) - computed as a two-term recursion over time instead of
 * an F-tap sum: about 10 operations per sample whatever F is.  causal != 0: the convolution of slayer_conv_f32;
 * causal == 0: the correlation of slayer_corr_f32.  The recursion serves rows of at most 512 samples in a 16-byte
 * aligned tensor of whole 16-byte vectors, and longer rows of whole vectors (T % 4 == 0) with F <= 256, which it
 * takes in pieces of 256 samples with the state carried from piece to piece.  `filt` must hold exactly that kernel:
 * it is what every other shape is filtered with (through the F-tap kernels), and what a tile of four rows that holds
 * a non-finite sample is filtered with (a long row: from the piece with that sample on), so that infinities and NaNs
 * reach the samples the reference lets them reach.  The caller states tau and mult.  The result agrees with the F-tap chain to
 * rounding, relative to the sum of the magnitudes of the terms of the UNTRUNCATED response
 * (sum_k |x[t -+ k]| |mult| (k Ts / tau) exp(1 - k Ts / tau) over all k): 1e-5 of that sum at most, about 1e-6
 * measured.  Optional: a caller that does not know its filter to be an alpha kernel keeps calling
 * slayer_conv_f32 / slayer_corr_f32.
 */
int slayer_psp_alpha_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T, int64_t F,
                         float tau, float mult, float Ts, int causal, void *stream);

/*
 * slayer_spike_bwd_corr_f32 for such an alpha kernel: the surrogate gradient of the spike function, applied to the
 * samples on their way in, then the correlation as that recursion - the backward pass of spike(psp(x)) (the
 * reference's MLP ordering, example/02_NMNIST_MLP/nmnistMLP.py:59-60; src/slayer.py:857-865 followed by :887-899)
 * in one kernel, 12 bytes per neuron-timestep.  Same bound as slayer_psp_alpha_f32 with
 * x = gradOut * (scale / tauRho) * exp(-|u - theta| / tauRho); tauRho here is the scaled time constant (the `tau`
 * of slayer_spike_bwd_f32).  Shapes outside the recursion's reach run slayer_spike_bwd_corr_f32.
 */
int slayer_spike_bwd_psp_alpha_f32(float *gradIn, const float *gradOut, const float *u, const float *filt,
                                   int64_t nNeurons, int64_t T, int64_t F, float tau, float mult, float theta,
                                   float tauRho, float scale, float Ts, void *stream);

/*
 * The other order of the same two operations, the backward pass of psp(spike(u)) - what every layer of the
 * reference's convolutional networks does with its spikes (example/03_NMNIST_CNN/nmnistCNN.py:55-60:
 * spike(conv(psp(spike(...))))): gradIn = pdf(u) * (corr(gradPsp) + gradSpike), i.e.
 * _pspFunction.backward (src/slayer.py:888-893) followed by _spikeFunction.backward (src/slayer.py:858-865)
 * in one kernel, without the intermediate tensor.  gradPsp is the gradient with respect to the PSP signal,
 * gradSpike (may be NULL) the gradient that reaches the spikes directly; filt, tau, mult as in
 * slayer_psp_alpha_f32, theta, tauRho, scale as in slayer_spike_bwd_f32.  Only as the recursion: shapes it
 * does not serve (see slayer_psp_alpha_f32) return SLAYER_EUNSUPPORTED, and the caller runs
 * slayer_corr_f32, adds, and runs slayer_spike_bwd_f32.
 */
int slayer_psp_spike_bwd_alpha_f32(float *gradIn, const float *gradPsp, const float *gradSpike, const float *u,
                                   const float *filt, int64_t nNeurons, int64_t T, int64_t F, float tau, float mult,
                                   float theta, float tauRho, float scale, float Ts, void *stream);

/*
 * Spike generation with the time shift that follows it fused into the store of the spikes.
 * Replaces the call pair slayerCuda.getSpikes (src/cuda/slayerKernels.cu:14-39) -> slayerCuda.shift
 * (src/cuda/slayerKernels.cu:77-134) that `delayShift(spike(u), d)` / `delay(spike(u))` make
 * (src/slayer.py:333-391, 901-979): 8 of the 20 bytes per sample of the two kernels are not moved.
 *
 * s[t] = spike[t - k] with k = (int)(d / delayTs) (0 where t - k is outside the row); d is
 * delayLut[neuron % lutSize] when delayLut is given (one delay per neuron of a batch item, nNeurons a
 * multiple of lutSize) and `delay` otherwise, of any size and sign.  `u` is updated in place and NOT shifted,
 * exactly as by slayer_get_spikes_f32.  Fused shapes: nuSize <= 24 and rows of at most 352 samples, or longer
 * rows of whole 16-byte vectors up to 16384 samples (those travel in pieces: the kernel keeps the spike bits
 * of the whole row and stores the shifted spikes behind the row's last piece).  Other shapes return
 * SLAYER_EUNSUPPORTED with nothing launched - call the two functions then.
 */
int slayer_get_spikes_delayed_f32(float *s, float *u, const float *nu, const float *delayLut,
                                  int64_t lutSize, float delay, float delayTs, int64_t nNeurons,
                                  int64_t T, int64_t nuSize, float theta, float Ts, void *stream);

/*
 * Backward pass of the above in one kernel: gradIn[t] = gradOut[t + k] * scale/tau * exp(-|u[t]-theta|/tau)
 * (0 where t + k is outside the row), i.e. the backward shift of _delayFunction / delayShift
 * (src/slayer.py:944-979) followed by the surrogate gradient of _spikeFunction.backward
 * (src/slayer.py:857-865), bit-identical to slayer_shift_*_f32 with the negated delay followed by
 * slayer_spike_bwd_f32.  Any T.
 */
int slayer_spike_bwd_delayed_f32(float *gradIn, const float *gradOut, const float *u,
                                 const float *delayLut, int64_t lutSize, float delay, float delayTs,
                                 int64_t nNeurons, int64_t T, float theta, float tau, float scale,
                                 void *stream);

/* Bytes of caller-provided device workspace that slayer_delay_grad_f32 needs (may be 0). */
int64_t slayer_delay_grad_workspace_bytes(int64_t nBatch, int64_t nPerBatch, int64_t T);

/*
 * Gradient with respect to a per-neuron delay table, fused into one pass plus a small
 * deterministic reduction.
 * Replaces the conv + multiply + sum of _delayFunction.backward (src/slayer.py:949-955).
 *
 * gradDelay[m] = Ts * sum_{b,t} gradOut[b][m][t] * (out[b][m][t-1] - out[b][m][t]) / Ts,
 * out[.][.][-1] = 0, for the [nBatch][nPerBatch][T] tensors `out` (the shifted signal) and
 * `gradOut`.  `workspace` must hold slayer_delay_grad_workspace_bytes(...) bytes.
 */
int slayer_delay_grad_f32(float *gradDelay, const float *out, const float *gradOut,
                          float *workspace, int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts,
                          void *stream);

/*
 * slayer_delay_grad_f32 for callers that cannot allocate device memory (code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc): it has no counterpart in the reference.  Same
 * arguments and bit-identical results, but the partial sums live in a fixed array inside the library's
 * device image (4 bytes per neuron row, slayer_delay_grad_static_max_rows() = 262144 rows = 1 MiB, held
 * by every GPU the library runs on until the process ends) instead of a caller workspace, so the call
 * allocates and frees nothing.  nBatch * nPerBatch beyond that maximum: SLAYER_EUNSUPPORTED, nothing
 * launched.  The array's device address is looked up on the first call on each device (make that call
 * outside a graph capture).  All calls on one GPU share the array: calls that overlap on one GPU (two
 * streams, two threads) race - serialise them.  Nothing needs clearing between calls.
 */
int64_t slayer_delay_grad_static_max_rows(void);
int slayer_delay_grad_static_f32(float *gradDelay, const float *out, const float *gradOut,
                                 int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts, void *stream);

/*
 * Loihi CUBA (current based) integer neuron.
 * Replaces slayerLoihiCuda.getSpikes -> getSpikesCuda (src/cuda/slayerLoihiKernels.cu:12-46),
 * kernel and launcher src/cuda/spikeLoihiKernels.h:9-96.
 *
 * Per neuron row, int32 state (current, voltage) starting at 0, weightScale = 1 << (6+wgtExp):
 *   t = 0 : s = v = u = 0, the input sample is ignored;
 *   t >= 1: current = decay(current, iDecay) + weightScale * (int)w[t]
 *           voltage = decay(voltage, vDecay) + current
 *           decay(x, d) = sign(x) * ((|x| * (4096 - d)) >> 12)      (32-bit wrap-around)
 *           spike = voltage > theta and the neuron is not refractory; a spike makes the neuron
 *           refractory until refDelay steps later; while refractory (and at the spike) the
 *           voltage carried to the next step is 0.
 *           s[t] = spike, u[t] = current, v[t] = spike ? vDecay : carried voltage.
 * Outputs are exact integers stored as float32, bit-identical to the sequential loop.
 * refDelay must be >= 1 (the reference reads an unwritten sample for 0): SLAYER_EINVAL.
 * wgtExp must satisfy 6 + wgtExp < 32.
 */
int slayer_loihi_get_spikes_f32(float *s, float *v, float *u, const float *w, int64_t nNeurons,
                                int64_t T, uint32_t wgtExp, int32_t theta, uint32_t iDecay,
                                uint32_t vDecay, uint32_t refDelay, void *stream);

/*
 * The same neuron with the time shift that follows it in Loihi networks fused in, and with
 * optional outputs.  Replaces the call pair spikeLoihi -> delayShift(spike, 1) of the reference's
 * network definitions (src/auto/loihi.py:67-69, exampleLoihi/03_IBMGesture/ibmGestureTrain.py:57-81):
 * slayerLoihiCuda.getSpikes (src/cuda/slayerLoihiKernels.cu:12-46) followed by slayerCuda.shift
 * (src/cuda/slayerKernels.cu:114-134).
 *
 * s[t] = spike[t - delaySteps] (0 for t < delaySteps), 0 <= delaySteps <= 31 (more:
 * SLAYER_EUNSUPPORTED - shift separately); v and u are as in slayer_loihi_get_spikes_f32 (not
 * shifted) and either may be NULL when the caller does not need it (the layer engine needs the
 * voltage for the backward pass only and never the current), which saves its 4 bytes per sample.
 */
int slayer_loihi_get_spikes_delayed_f32(float *s, float *v, float *u, const float *w,
                                        int64_t nNeurons, int64_t T, uint32_t wgtExp, int32_t theta,
                                        uint32_t iDecay, uint32_t vDecay, uint32_t refDelay,
                                        int32_t delaySteps, void *stream);

/*
 * ---- Per-timestep synapses ---------------------------------------------------------------------
 * The reference's conv / pool / convTranspose / unpool layers apply a 2-D filter over (H, W) to
 * every time sample of an [N][C][H][W][T] tensor by calling torch's conv3d / conv_transpose3d
 * with a kernel of time extent 1 (src/slayer.py:499-507, :565-575, :631-643, :732-748).  The three
 * entry points below are that operation and its two gradients on T-innermost tensors; the pooling
 * layers are the case C = O = 1 on the tensor reshaped to [N][1][C*H][W][T], the transposed layers
 * use the input gradient as their forward pass.
 *
 * Geometry: input [N][C][H][W][T], weights [O][C/groups][KH][KW] (the reference's trailing
 * time extent of 1 dropped), output [N][O][OH][OW][T] with
 * OH = (H + 2*padH - dilH*(KH-1) - 1) / strideH + 1 (0 when the filter does not fit), OW alike.
 * One batch item of the input and of the output must stay below 2 GiB (SLAYER_EUNSUPPORTED).
 *
 * Arithmetic: fp32 sums; the order of the additions depends on the geometry, not on the launch (no
 * atomics).  The forward pass of layers with at least 16 output channels and about 100 or more taps
 * per output, and the weight gradient of layers large enough for the matrix cores, multiply on bf16
 * matrix instructions over operands split into three bf16 parts each (six of the nine partial
 * products; three when the input holds nothing below the upper 16 bits of its numbers, as spike
 * tensors do): every result within 1e-6 of the sum of its terms' magnitudes.  Parts below 2^-126 are
 * flushed to zero, and a non-finite input sample gives NaN where an fp32 sum may give an infinity.
 */
typedef struct slayer_synapse_geom {
    int32_t N, C, H, W, T;
    int32_t O, KH, KW;
    int32_t strideH, strideW, padH, padW, dilH, dilW, groups;
} slayer_synapse_geom;

/* Validates the geometry and returns the output extents (either pointer may be NULL). */
int slayer_synapse_out_shape(const slayer_synapse_geom *geom, int32_t *OH, int32_t *OW);

/*
 * out[n][o][a][b][t] = sum_{c in group(o), i, j} weight[o][c'][i][j] *
 *                      in[n][c][a*strideH - padH + i*dilH][b*strideW - padW + j*dilW][t]
 * (samples outside the input count as 0).  Replaces F.conv3d in _convLayer.forward
 * (src/slayer.py:499-507) and _poolLayer.forward (src/slayer.py:565-575).
 */
int slayer_synapse_conv_f32(float *out, const float *in, const float *weight,
                            const slayer_synapse_geom *geom, void *stream);

/*
 * Gradient of slayer_synapse_conv_f32 with respect to `in` (every element of gradIn is written).
 * Replaces the input gradient autograd derives for F.conv3d in those layers, and is the forward
 * pass F.conv_transpose3d of _convTransposeLayer / _unpoolLayer (src/slayer.py:631-643, :732-748),
 * whose weight tensor [inChannels][outChannels/groups][KH][KW] is the weight tensor of the
 * convolution it transposes.
 */
int slayer_synapse_conv_grad_input_f32(float *gradIn, const float *gradOut, const float *weight,
                                       const slayer_synapse_geom *geom, void *stream);

/* Bytes of caller-provided device workspace for slayer_synapse_conv_grad_weight_f32 (may be 0). */
int64_t slayer_synapse_conv_grad_weight_workspace_bytes(const slayer_synapse_geom *geom);

/*
 * gradW[o][c'][i][j] = sum_{n,a,b,t} gradOut[n][o][a][b][t] *
 *                      in[n][c][a*strideH - padH + i*dilH][b*strideW - padW + j*dilW][t]
 * Replaces the weight gradient autograd derives for F.conv3d / F.conv_transpose3d in the same
 * layers.  Partial sums go through `workspace` and are added in a fixed order (deterministic).
 */
int slayer_synapse_conv_grad_weight_f32(float *gradW, const float *gradOut, const float *in,
                                        float *workspace, const slayer_synapse_geom *geom,
                                        void *stream);

/*
 * ---- Fully connected synapse on sparse input ---------------------------------------------------
 * out[n][o][t] = sum_k weight[o][k] * x[n][k][t], summed over the non-zero x only, in ascending k: the
 * product of _denseLayer.forward (src/slayer.py:435-440: an F.conv3d whose kernel spans the whole
 * (C, H, W) extent of the input, i.e. per batch item the matrix product W[O x K] * x[K x T] with
 * K = C*H*W) for inputs that are spike tensors.  x is [N][K][T], weight [O][K], out [N][O][T] (every
 * element is written).  Four launches: x is transposed to [N][T][K] and weight to [K][O], so that a
 * column (n, t) of x is a contiguous row whose events fetch contiguous rows of the weights; one wavefront
 * per column (and slice of the input channels) sums its events; the slices are added and the result goes
 * back to [N][O][T].  `workspace` holds slayer_dense_events_workspace_bytes(N, K, O, T) bytes.  The result
 * is the dense product up to the order of the additions, and without the 0 * inf = NaN terms a dense
 * product has when weights are not finite.  The work grows with the number of non-zero inputs: above a
 * few per cent, or with few input channels, a library matrix product is faster, and the caller chooses.
 * O <= 1024, N <= 65535, weight below 2 GiB, else SLAYER_EUNSUPPORTED.
 */
int64_t slayer_dense_events_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T);
int slayer_dense_events_f32(float *out, const float *x, const float *weight, float *workspace, int64_t N,
                            int64_t K, int64_t O, int64_t T, void *stream);

/*
 * gradW[o][k] = sum_{n,t} gradOut[n][o][t] * x[n][k][t], summed over the non-zero x only, in ascending
 * (n, t): the weight gradient of _denseLayer (src/slayer.py:393-440: an F.conv3d whose kernel spans the
 * whole (C, H, W) extent of the input, i.e. per batch item the matrix product W[O x K] * x[K x T] with
 * K = C*H*W; replaces the weight gradient autograd derives for that call) for inputs that are spike
 * tensors.  x is [N][K][T], gradOut [N][O][T], gradW [O][K] (every element is written).  Three launches:
 * gradOut is transposed to [N][T][O], so that an event fetches one contiguous row; one wavefront per
 * input channel and slice of the batch's samples sums its events; the slices are added in a fixed
 * order.  `workspace` holds slayer_dense_events_grad_weight_workspace_bytes(N, K, O, T) bytes.  The result
 * is the dense product up to the order of the additions, and without the 0 * inf = NaN terms a dense
 * product has when gradients are not finite.  The work grows with the number of non-zero inputs: above a
 * few per cent, or with few input channels, a library matrix product is faster, and the caller chooses.
 * O <= 1024, N <= 65535, and gradOut must stay below 2 GiB, else SLAYER_EUNSUPPORTED.
 */
int64_t slayer_dense_events_grad_weight_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T);
int slayer_dense_events_grad_weight_f32(float *gradW, const float *gradOut, const float *x,
                                        float *workspace, int64_t N, int64_t K, int64_t O, int64_t T,
                                        void *stream);

/*
 * ---- Fully connected synapse with few inputs, on the matrix cores --------------------------------
 * out[n][o][t] = sum_{k<K} W[o][k] * x[n][k][t] with W[o][k] = w[o * wRow + k * wCol]: per batch item the
 * matrix product W[O x K] * x[K x T] of _denseLayer.forward (src/slayer.py:435-440, see above) with
 * wRow = K, wCol = 1, and its input gradient W^T * gradOut (the one autograd derives for that call) with
 * w the same weight, wRow = 1, wCol = the layer's input count, and the roles of K and O exchanged.  x is
 * [N][K][T], out [N][O][T] (every element is written); T a multiple of 4, x and out 16-byte aligned, K * T
 * and O * T below 2^29, else SLAYER_EUNSUPPORTED (slayer_dense_rows_supported says so beforehand).
 * `workspace` holds slayer_dense_rows_workspace_bytes(K, O) bytes, 16-byte aligned (the weights, split).
 * One launch per 224 inputs (and a small one that splits the weights): the rows of W stay in registers, split into three bf16 parts each, the tiles of
 * x are split on their way into LDS, and the products run on bf16 matrix instructions (six of the nine partial
 * products, each exact in the fp32 accumulator; three when a tile of x holds spikes, i.e. values with at most 8
 * significant bits).  The result is the product up to the order of the additions and 2^-23 of each term: within
 * 1e-6 of sum_k |W[o][k]| |x[n][k][t]|.  Weights and samples must be finite.  Meant for layers with up to a
 * few hundred inputs, where a library product spends its time on fp32 matrix instructions.
 */
int slayer_dense_rows_supported(int64_t N, int64_t K, int64_t O, int64_t T);
int64_t slayer_dense_rows_workspace_bytes(int64_t K, int64_t O);
int slayer_dense_rows_f32(float *out, const float *w, const float *x, void *workspace, int64_t N, int64_t K, int64_t O,
                          int64_t T, int64_t wRow, int64_t wCol, void *stream);

/*
 * gradW[o][k] = sum_{n,t} gradOut[n][o][t] * x[n][k][t]: the weight gradient of the same layers (the one autograd
 * derives for the F.conv3d of _denseLayer.forward, src/slayer.py:435-440), for up to 448 inputs and 256 outputs.
 * x is [N][K][T], gradOut [N][O][T], gradW [O][K] (every element is written); T a multiple of 4, both tensors
 * 16-byte aligned.  `workspace` holds slayer_dense_rows_grad_weight_workspace_bytes(N, K, O, T) bytes: every
 * work-group sums a range of the batch's samples for all weights - on bf16 matrix instructions over split operands,
 * as slayer_dense_rows_f32 - and a second launch adds the work-groups' sums in a fixed order.  Within 1e-6 of
 * sum_{n,t} |gradOut| |x|.
 */
int slayer_dense_rows_grad_weight_supported(int64_t N, int64_t K, int64_t O, int64_t T);
int64_t slayer_dense_rows_grad_weight_workspace_bytes(int64_t N, int64_t K, int64_t O, int64_t T);
int slayer_dense_rows_grad_weight_f32(float *gradW, const float *gradOut, const float *x, void *workspace, int64_t N,
                                      int64_t K, int64_t O, int64_t T, void *stream);

/*
 * ---- Weight quantisation of the Loihi layers ---------------------------------------------------
 * out[i] = round(in[i] / step) * step the way torch evaluates the expression on the GPU for a Python number
 * `step`: in[i] times the fp32 rounding of the double-precision reciprocal of step, to the nearest integer with
 * ties to even, times the fp32 rounding of step: quantizeWeights.forward
 * (src/quantizeParams.py:17-23), which the Loihi layers apply to their weights in every forward pass
 * (src/slayerLoihi.py:124-139), in one launch.  n <= 2^32 elements; out may be in.
 */
int slayer_quantize_f32(float *out, const float *in, int64_t n, double step, void *stream);

/*
 * ---- Spike event files to spike tensors -------------------------------------------------------
 * Decodes packed spike events and bins them into spike tensors, one launch for a batch of samples.
 * Replaces spikeFileIO.read1Dspikes / read2Dspikes / read3Dspikes (src/spikeFileIO.py:162-184,
 * :233-259, :296-321) followed by event.toSpikeTensor (src/spikeFileIO.py:66-144), which the
 * reference runs with numpy in data-loader workers before copying a dense tensor to the GPU.
 *
 * bytes: the samples' file contents back to back on the device (nBytes in all); format 1 = 5-byte
 * events (16-bit neuron id, polarity bit, 23-bit time in us), 2 = 5-byte events (x, y, polarity bit,
 * 23-bit time), 3 = 7-byte events (12-bit x, 12-bit y, 8-bit channel, 24-bit time).
 * sampleTable: device array [nSamples][3] = {first byte of the sample, number of events, time shift
 * in bins}; an entry that does not lie inside the buffer is skipped.  maxEvents: the largest event
 * count in the table (sizes the launch).  tensor: [nSamples][C][H][W][T].
 * Per event: polarity minus the smallest polarity of its sample, bin = rint((time in ms) /
 * samplingTime) - shift in double precision; events outside the tensor are dropped; mode 0 ("OR")
 * stores 1/samplingTime, mode 1 ("SUM") stores base[...] + 1/samplingTime, where `base` is a copy of
 * the tensor from before the call (required and distinct from `tensor` in mode 1, ignored in
 * mode 0) - once per bin however many events share it, like numpy's indexed +=.
 */
int slayer_bin_packed_events_f32(float *tensor, const float *base, const uint8_t *bytes, int64_t nBytes,
                                 const int64_t *sampleTable, int64_t nSamples, int64_t maxEvents,
                                 int32_t format, int32_t C, int32_t H, int32_t W, int32_t T,
                                 double samplingTime, int32_t mode, void *stream);

/*
 * The binning alone, for one sample whose events are already decoded: x, y (NULL = all 0), p as
 * int32 and the time in milliseconds as double, tensor [C][H][W][T].  Replaces
 * event.toSpikeTensor (src/spikeFileIO.py:66-144) for events that did not come from a file.
 */
int slayer_bin_events_f32(float *tensor, const float *base, const int32_t *x, const int32_t *y,
                          const int32_t *p, const double *tMs, int64_t nEvents, int64_t timeShift,
                          int32_t C, int32_t H, int32_t W, int32_t T, double samplingTime,
                          int32_t mode, void *stream);

/*
 * ---- Spike-train loss ---------------------------------------------------------------------------
 * error = psp(out - desired) [+ addend], loss = 1/2 * sum(error^2) * Ts in two launches.
 * Replaces the tensor expressions of spikeLoss.spikeTime (src/spikeLoss.py:56-58) and of the last
 * two statements of spikeLoss.numSpikes (src/spikeLoss.py:100-104, where `addend` is the spike count
 * error inside the target region).  out, desired, error and the optional addend are [rows][T]; psp
 * is the causal filter of slayer_conv_f32 with the same arithmetic; `loss` is one float.  The sum
 * has a fixed association (deterministic).  `workspace` holds slayer_spike_loss_workspace_bytes(rows)
 * bytes.  Rows whose T + 2 F floats exceed 60 KB return SLAYER_EUNSUPPORTED (nothing launched).
 */
int64_t slayer_spike_loss_workspace_bytes(int64_t rows);
int slayer_spike_loss_f32(float *loss, float *error, const float *out, const float *desired,
                          const float *addend, const float *srm, float *workspace, int64_t rows,
                          int64_t T, int64_t F, float Ts, void *stream);

#ifdef __cplusplus
}
#endif

#endif /* SLAYER_HIP_H_INCLUDED */

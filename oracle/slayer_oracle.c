/*
 * CPU oracle for SLAYER's per-neuron temporal kernels.
 *
 * TEST INFRASTRUCTURE ONLY.  This file restates, in plain C, the arithmetic of the
 * reference's CUDA kernels so that the HIP kernels can be checked against it.  Nothing in
 * the product path may link, load or call it; only the test-suite, the smoke check and the
 * benchmark's cpu_baseline leg do.
 *
 * Every tensor is a dense row-major [nNeurons][T] float32 array ("neuron row" = T
 * consecutive samples of one neuron).  All functions are independent per row, so the
 * optional OpenMP parallel-for over rows does not change any result.
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off: the compiler must not fuse
 * multiply-adds on its own; where a fused multiply-add is wanted it is written as fmaf()).
 *
 * Parity pins (what fixes each function besides this restatement) are listed per function.
 */
#include <math.h>
#include <stdint.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

static int g_threads = 1;

/* Number of host threads used for the row loop (1 = scalar port). */
void oracle_set_threads(int n) { g_threads = n < 1 ? 1 : n; }
int oracle_get_threads(void) { return g_threads; }
int oracle_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------
 * SRM spike generation.  Follows src/cuda/spikeKernels.h:9-38 (getSpikesKernel) and the
 * shape convention of src/cuda/slayerKernels.cu:14-39.
 *
 * For every neuron row, walking t = 0 .. T-1 in order: when u[t] >= theta (note: >=) the
 * output spike is 1/Ts and the refractory kernel nu[0 .. nuSize-1] is added onto
 * u[t .. t+nuSize-1] (clipped at T, tap 0 included); otherwise the output is 0.  u is
 * updated in place, one fp32 add per tap, in the time order of the spikes that cause them.
 *
 * Pins: reference-held (u_before, u_after, spike) triples snnData/spikeFunc{Hid,Hid04,Out}.txt;
 * brute-force numpy loop of test/test_slayer002.py:154-167; special cases (theta = +inf,
 * single supra-threshold sample).
 * ---------------------------------------------------------------------------------------- */
void oracle_get_spikes_f32(float *s, float *u, const float *nu, int64_t nNeurons, int64_t T,
                           int64_t nuSize, float theta, float Ts)
{
    const float amplitude = 1.0f / Ts;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t n = 0; n < nNeurons; ++n) {
        float *ur = u + n * T;
        float *sr = s + n * T;
        for (int64_t t = 0; t < T; ++t) {
            if (ur[t] >= theta) {
                sr[t] = amplitude;
                int64_t last = (t + nuSize <= T) ? nuSize : (T - t);
                for (int64_t j = 0; j < last; ++j) ur[t + j] += nu[j];
            } else {
                sr[t] = 0.0f;
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Causal temporal convolution (psp forward).  Follows src/cuda/convKernels.h:10-35:
 *     out[n,t] = Ts * sum_{i=0..F-1, t-i>=0} in[n,t-i] * filt[i]
 * accumulated in fp32 starting from 0 in tap order i = 0,1,2,..., multiplied by Ts after the
 * sum.  fused != 0 evaluates every step as one fmaf(in, filt, acc) (what a GPU compiler
 * makes of `acc += a*b`); fused == 0 rounds the product and the sum separately.
 *
 * Pins: equals numpy.convolve(x, filt)[:T]*Ts and a left-padded conv3d with the flipped
 * filter (test/test_slayer011.py:39-43); golden torch_validate/forward_prop/s1.csv -> a1.csv,
 * back_prop/des_s.csv -> des_a.csv, input_validate/1_binned_spikes.csv ->
 * torch_validate/1_spike_response_signal.csv; impulse response; linearity.
 * ---------------------------------------------------------------------------------------- */
__attribute__((target_clones("fma", "default")))
void oracle_conv_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T,
                     int64_t F, float Ts, int fused)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t n = 0; n < nNeurons; ++n) {
        const float *x = in + n * T;
        float *y = out + n * T;
        for (int64_t t = 0; t < T; ++t) {
            float acc = 0.0f;
            int64_t taps = (t + 1 < F) ? (t + 1) : F;
            if (fused) {
                for (int64_t i = 0; i < taps; ++i) acc = fmaf(x[t - i], filt[i], acc);
            } else {
                for (int64_t i = 0; i < taps; ++i) {
                    float p = x[t - i] * filt[i];
                    acc = acc + p;
                }
            }
            y[t] = acc * Ts;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Anti-causal temporal correlation (psp backward).  Follows src/cuda/convKernels.h:37-62:
 *     out[n,t] = Ts * sum_{i=0..F-1, t+i<T} in[n,t+i] * filt[i]
 * same accumulation rules as the convolution.  It is the adjoint of oracle_conv_f32.
 *
 * Pins: adjoint identity <conv(x),y> = <x,corr(y)>; numpy.correlate slice; joint
 * forward/backward golden gradients snnData/gradW{1,2}Initial.txt.
 * ---------------------------------------------------------------------------------------- */
__attribute__((target_clones("fma", "default")))
void oracle_corr_f32(float *out, const float *in, const float *filt, int64_t nNeurons, int64_t T,
                     int64_t F, float Ts, int fused)
{
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t n = 0; n < nNeurons; ++n) {
        const float *x = in + n * T;
        float *y = out + n * T;
        for (int64_t t = 0; t < T; ++t) {
            float acc = 0.0f;
            int64_t taps = (T - t < F) ? (T - t) : F;
            if (fused) {
                for (int64_t i = 0; i < taps; ++i) acc = fmaf(x[t + i], filt[i], acc);
            } else {
                for (int64_t i = 0; i < taps; ++i) {
                    float p = x[t + i] * filt[i];
                    acc = acc + p;
                }
            }
            y[t] = acc * Ts;
        }
    }
}

/* Number of whole sampling steps in a delay: C cast of the fp32 quotient, i.e. truncation
 * toward zero (src/cuda/shiftKernels.h:24,51).  Out-of-range quotients saturate, NaN -> 0,
 * which is what the GPU conversion instruction does. */
static int32_t steps_of(float delay, float Ts)
{
    float q = delay / Ts;
    if (q != q) return 0;
    if (q >= 2147483648.0f) return INT32_MAX;
    if (q <= -2147483648.0f) return INT32_MIN;
    return (int32_t)q;
}

/* ------------------------------------------------------------------------------------------
 * Time shift.  Follows src/cuda/shiftKernels.h:9-61 and the dispatch of
 * src/cuda/slayerKernels.cu:77-134.
 *     k = (int)(d / Ts);  out[n,t] = (0 <= t-k < T) ? in[n,t-k] : 0
 * lutSize == 1: the single delay lut[0] applies to every row.
 * lutSize == nPerBatch: row (b, m) uses lut[m]; the table is shared by all nBatch batches.
 *
 * Pins: exact equality with slicing by int(d/Ts) for positive, zero and negative delays
 * (test/test_slayer009.py:29-63); shift(shift(x,d),-d) restores the interior.
 * ---------------------------------------------------------------------------------------- */
void oracle_shift_f32(float *out, const float *in, const float *lut, int64_t lutSize,
                      int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts)
{
    const int64_t rows = nBatch * nPerBatch;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float d = (lutSize == 1) ? lut[0] : lut[r % nPerBatch];
        int64_t k = steps_of(d, Ts);
        const float *x = in + r * T;
        float *y = out + r * T;
        for (int64_t t = 0; t < T; ++t) {
            int64_t src = t - k;
            y[t] = (src >= 0 && src < T) ? x[src] : 0.0f;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Spike-function surrogate gradient.  Follows _spikeFunction.backward, src/slayer.py:857-865
 * (and the unused native evalRhoKernel, src/cuda/spikeKernels.h:41-52):
 *     gradIn = gradOut * ( scale/tau * exp( -|u - theta| / tau ) ),  tau = tauRho*theta
 * with the same fp32 operation order as the torch expression (scale/tau first, then the
 * exponential of the fp32 quotient, product, product).
 *
 * Pins: closed form in fp64; torch_validate/back_prop/rho3.csv against forward_prop/u3.csv
 * with pdf_params {scale 1, tau 4.3429}.
 * ---------------------------------------------------------------------------------------- */
void oracle_spike_bwd_f32(float *gradIn, const float *gradOut, const float *u, float theta,
                          float tau, float scale, int64_t numel)
{
    const float gain = scale / tau;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t i = 0; i < numel; ++i) {
        float d = fabsf(u[i] - theta);
        float pdf = gain * expf(-d / tau);
        gradIn[i] = gradOut[i] * pdf;
    }
}

/* ------------------------------------------------------------------------------------------
 * Delay gradient.  Follows _delayFunction.backward, src/slayer.py:949-955:
 *     diff[n,t]   = out[n,t]*(-1/Ts) + out[n,t-1]*(1/Ts)      (2-tap causal conv, out[-1] = 0)
 *     gradDelay[m] = Ts * sum_{b,t} gradOut[b,m,t] * diff[b,m,t]
 * The per-element values are fp32 as in the reference; the reduction is carried in fp64 so
 * that the oracle is independent of summation order.
 *
 * Pins: manual formula of test/test_slayer010.py:73-80 (-sum(e * d(psp)/dt) * Ts).
 * ---------------------------------------------------------------------------------------- */
void oracle_delay_grad_f32(float *gradDelay, const float *out, const float *gradOut,
                           int64_t nBatch, int64_t nPerBatch, int64_t T, float Ts)
{
    const float f0 = -1.0f / Ts, f1 = 1.0f / Ts;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t m = 0; m < nPerBatch; ++m) {
        double acc = 0.0;
        for (int64_t b = 0; b < nBatch; ++b) {
            const float *y = out + (b * nPerBatch + m) * T;
            const float *g = gradOut + (b * nPerBatch + m) * T;
            for (int64_t t = 0; t < T; ++t) {
                float d = y[t] * f0;
                if (t > 0) d = d + y[t - 1] * f1;
                acc += (double)(g[t] * d);
            }
        }
        gradDelay[m] = (float)(acc * (double)Ts);
    }
}

/* float -> int32 the way the GPU converts: toward zero, saturating, NaN -> 0. */
static int32_t trunc_sat(float x)
{
    if (x != x) return 0;
    if (x >= 2147483648.0f) return INT32_MAX;
    if (x <= -2147483648.0f) return INT32_MIN;
    return (int32_t)x;
}

/* Sign-magnitude decay of a Loihi state variable: the magnitude is scaled by
 * (4096 - decay)/4096 with the fraction dropped, so the state moves toward zero.  All
 * products are 32-bit unsigned (wrap-around) and the shift is logical, which is what the C
 * promotion rules make of src/cuda/spikeLoihiKernels.h:47-48. */
static uint32_t loihi_decay(int32_t state, uint32_t decay)
{
    uint32_t sign = (state >= 0) ? 1u : 0xFFFFFFFFu;
    uint32_t magnitude = sign * (uint32_t)state;
    uint32_t scaled = (magnitude * (4096u - decay)) >> 12;
    return sign * scaled;
}

/* ------------------------------------------------------------------------------------------
 * Loihi CUBA neuron.  Follows src/cuda/spikeLoihiKernels.h:9-72,95 and
 * src/cuda/slayerLoihiKernels.cu:12-46.
 *   t = 0: all three outputs are 0 and the input sample is ignored.
 *   t >= 1: current = decay(current, iDecay) + (1 << (6+wgtExp)) * (int)w[t]
 *           voltage = decay(voltage, vDecay) + current
 *           if t >= refDelay: refState -= (spike written at t - refDelay)
 *           spike   = voltage > theta (signed, strict) and refState == 0
 *           voltage kept for the next step = 0 if spike or refState != 0, else voltage
 *           refState += spike
 *           outputs: s = spike, u = current, v = spike ? vDecay : kept voltage
 * refDelay == 0 reads an unwritten sample in the reference; it is rejected by the caller.
 *
 * Pins: numpy Neuron.run of test/test_slayerLoihi002.py:30-82 (refDelay 2..17); Loihi-chip
 * recordings test_files/Loihi/LoihiData; closed-form impulse response (twice the Loihi
 * PSP kernel: 128, 220, 285, 330, ...) = second row of LoihiData/LoihiVth05.txt.
 * ---------------------------------------------------------------------------------------- */
void oracle_loihi_get_spikes_f32(float *s, float *v, float *u, const float *w, int64_t nNeurons,
                                 int64_t T, uint32_t wgtExp, int32_t theta, uint32_t iDecay,
                                 uint32_t vDecay, uint32_t refDelay)
{
    const uint32_t weightScale = 1u << (6 + wgtExp);
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t n = 0; n < nNeurons; ++n) {
        const float *wr = w + n * T;
        float *sr = s + n * T, *vr = v + n * T, *ur = u + n * T;
        int32_t current = 0, voltage = 0;
        uint32_t refState = 0;
        for (int64_t t = 0; t < T; ++t) {
            if (t == 0) {
                sr[0] = 0.0f; vr[0] = 0.0f; ur[0] = 0.0f;
                continue;
            }
            int32_t cNew = (int32_t)(loihi_decay(current, iDecay) +
                                     weightScale * (uint32_t)trunc_sat(wr[t]));
            int32_t vNew = (int32_t)(loihi_decay(voltage, vDecay) + (uint32_t)cNew);
            if ((uint64_t)t >= refDelay) refState -= (uint32_t)sr[t - refDelay];
            uint32_t spike = (vNew > theta) && (refState == 0);
            voltage = (spike || refState != 0) ? 0 : vNew;
            refState += spike;
            current = cNew;
            sr[t] = (float)spike;
            ur[t] = (float)cNew;
            vr[t] = spike ? (float)(int32_t)vDecay : (float)voltage;
        }
    }
}

/* ------------------------------------------------------------------------------------------
 * Per-timestep synapse (2-D cross-correlation applied to every time sample of an
 * [N][C][H][W][T] tensor).  The reference's layers call torch's conv3d / conv_transpose3d with
 * a kernel of time extent 1 (src/slayer.py:441-449 dense, :499-507 conv, :565-575 pool,
 * :631-643 convTranspose, :732-748 unpool); this restates that operation's definition:
 *
 *   out[n][o][a][b][t] = sum_{c in group(o), i, j} w[o][c'][i][j] *
 *                        in[n][c][a*sH - pH + i*dH][b*sW - pW + j*dW][t]   (0 outside the tensor)
 *
 * with c' = c - group(o)*C/groups.  Sums are accumulated in double and rounded once, so the
 * result does not depend on a summation order.  geom = {N, C, H, W, T, O, KH, KW, sH, sW, pH, pW,
 * dH, dW, groups}.
 * Pins: torch.nn.functional.conv3d / conv_transpose3d and their autograd on the CPU (the very
 * routine the reference's layers call), the shift-and-add constructions of the reference's
 * tests (test/test_slayer007.py:36-48, :60-66, test/test_slayer013.py), adjoint identities.
 * ------------------------------------------------------------------------------------------ */
typedef struct {
    int32_t N, C, H, W, T, O, KH, KW, sH, sW, pH, pW, dH, dW, groups;
} oracle_synapse_geom;

static int64_t syn_out_extent(int64_t in, int64_t k, int64_t s, int64_t p, int64_t d)
{
    const int64_t span = in + 2 * p - d * (k - 1) - 1;
    return span < 0 ? 0 : span / s + 1;
}

void oracle_synapse_out_shape(const oracle_synapse_geom *g, int64_t *OH, int64_t *OW)
{
    *OH = syn_out_extent(g->H, g->KH, g->sH, g->pH, g->dH);
    *OW = syn_out_extent(g->W, g->KW, g->sW, g->pW, g->dW);
}

void oracle_synapse_conv_f32(float *out, const float *in, const float *w, const oracle_synapse_geom *g)
{
    int64_t OH, OW;
    oracle_synapse_out_shape(g, &OH, &OW);
    const int64_t Cg = g->C / g->groups, Og = g->O / g->groups, T = g->T;
    const int64_t rows = (int64_t)g->N * g->O * OH * OW;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const int64_t b = r % OW, a = (r / OW) % OH, o = (r / (OW * OH)) % g->O, n = r / (OW * OH * g->O);
        const int64_t grp = o / Og;
        for (int64_t t = 0; t < T; ++t) {
            double acc = 0.0;
            for (int64_t cl = 0; cl < Cg; ++cl)
                for (int64_t i = 0; i < g->KH; ++i)
                    for (int64_t j = 0; j < g->KW; ++j) {
                        const int64_t y = a * g->sH - g->pH + i * g->dH, x = b * g->sW - g->pW + j * g->dW;
                        if (y < 0 || y >= g->H || x < 0 || x >= g->W) continue;
                        const int64_t c = grp * Cg + cl;
                        acc += (double)w[((o * Cg + cl) * g->KH + i) * g->KW + j] *
                               (double)in[(((n * g->C + c) * g->H + y) * g->W + x) * T + t];
                    }
            out[r * T + t] = (float)acc;
        }
    }
}

/* Gradient of oracle_synapse_conv_f32 with respect to its input (= the transposed convolution
 * of gradOut): every product of the forward sum is sent back to the input sample it read. */
void oracle_synapse_conv_grad_input_f32(float *gradIn, const float *gradOut, const float *w,
                                        const oracle_synapse_geom *g)
{
    int64_t OH, OW;
    oracle_synapse_out_shape(g, &OH, &OW);
    const int64_t Cg = g->C / g->groups, Og = g->O / g->groups, T = g->T;
    const int64_t rows = (int64_t)g->N * g->C * g->H * g->W;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const int64_t x = r % g->W, y = (r / g->W) % g->H, c = (r / ((int64_t)g->W * g->H)) % g->C,
                      n = r / ((int64_t)g->W * g->H * g->C);
        const int64_t grp = c / Cg, cl = c % Cg;
        for (int64_t t = 0; t < T; ++t) {
            double acc = 0.0;
            for (int64_t ol = 0; ol < Og; ++ol)
                for (int64_t i = 0; i < g->KH; ++i)
                    for (int64_t j = 0; j < g->KW; ++j) {
                        const int64_t ya = y + g->pH - i * g->dH, xb = x + g->pW - j * g->dW;
                        if (ya < 0 || xb < 0 || ya % g->sH || xb % g->sW) continue;
                        const int64_t a = ya / g->sH, b = xb / g->sW;
                        if (a >= OH || b >= OW) continue;
                        const int64_t o = grp * Og + ol;
                        acc += (double)w[((o * Cg + cl) * g->KH + i) * g->KW + j] *
                               (double)gradOut[(((n * g->O + o) * OH + a) * OW + b) * T + t];
                    }
            gradIn[r * T + t] = (float)acc;
        }
    }
}

/* Gradient of oracle_synapse_conv_f32 with respect to the weights. */
void oracle_synapse_conv_grad_weight_f32(float *gradW, const float *gradOut, const float *in,
                                         const oracle_synapse_geom *g)
{
    int64_t OH, OW;
    oracle_synapse_out_shape(g, &OH, &OW);
    const int64_t Cg = g->C / g->groups, Og = g->O / g->groups, T = g->T;
    const int64_t nW = (int64_t)g->O * Cg * g->KH * g->KW;
#pragma omp parallel for num_threads(g_threads) schedule(static)
    for (int64_t q = 0; q < nW; ++q) {
        const int64_t j = q % g->KW, i = (q / g->KW) % g->KH, cl = (q / ((int64_t)g->KW * g->KH)) % Cg,
                      o = q / ((int64_t)g->KW * g->KH * Cg);
        const int64_t c = (o / Og) * Cg + cl;
        double acc = 0.0;
        for (int64_t n = 0; n < g->N; ++n)
            for (int64_t a = 0; a < OH; ++a) {
                const int64_t y = a * g->sH - g->pH + i * g->dH;
                if (y < 0 || y >= g->H) continue;
                for (int64_t b = 0; b < OW; ++b) {
                    const int64_t x = b * g->sW - g->pW + j * g->dW;
                    if (x < 0 || x >= g->W) continue;
                    const float *gp = gradOut + (((n * g->O + o) * OH + a) * OW + b) * T;
                    const float *ip = in + (((n * g->C + c) * g->H + y) * g->W + x) * T;
                    for (int64_t t = 0; t < T; ++t) acc += (double)gp[t] * (double)ip[t];
                }
            }
        gradW[q] = (float)acc;
    }
}

/* ------------------------------------------------------------------------------------------
 * Spike event files and event binning.  Follows src/spikeFileIO.py:
 *   read1Dspikes :162-184 (5 bytes: neuron id 16 bit, polarity 1 bit, time 23 bit in us),
 *   read2Dspikes :233-259 (5 bytes: x 8 bit, y 8 bit, polarity 1 bit, time 23 bit in us),
 *   read3Dspikes :296-321 (7 bytes: x 12 bit, y 12 bit, channel 8 bit, time 24 bit in us),
 *   event.__init__ :33 (the polarity is shifted so that its minimum over the events is 0),
 *   event.toSpikeTensor :66-144 (bin = round-half-even((t in ms) / samplingTime) - shift; events
 *   outside the tensor are dropped; 'OR' stores 1/samplingTime, 'SUM' stores the value the tensor
 *   held before the call plus 1/samplingTime - once, however many events share the bin, which is
 *   what numpy's indexed += does).
 * Pins: the reference's own sample triple test/test_files/NMNISTsmall/1.bs2 <->
 * input_validate/1_raw_spikes.csv <-> 1_binned_spikes.csv / 1_binned_spikes_ts2.csv (the csv
 * tensors were binned by truncation, so they pin decode, layout, validity and value on times
 * moved to the start of their bin), numpy.round / numpy.rint for the rounding itself.
 * ------------------------------------------------------------------------------------------ */
void oracle_decode_events(int32_t *x, int32_t *y, int32_t *p, int32_t *tUs, const uint8_t *bytes,
                          int64_t nEvents, int32_t format)
{
    for (int64_t e = 0; e < nEvents; ++e) {
        const uint8_t *b = bytes + e * (format == 3 ? 7 : 5);
        if (format == 1) {
            x[e] = (b[0] << 8) | b[1];
            y[e] = 0;
            p[e] = b[2] >> 7;
            tUs[e] = ((b[2] << 16) | (b[3] << 8) | b[4]) & 0x7FFFFF;
        } else if (format == 2) {
            x[e] = b[0];
            y[e] = b[1];
            p[e] = b[2] >> 7;
            tUs[e] = ((b[2] << 16) | (b[3] << 8) | b[4]) & 0x7FFFFF;
        } else {
            x[e] = (b[0] << 4) | (b[1] >> 4);
            y[e] = b[2] | ((b[1] & 0x0F) << 8);
            p[e] = b[3];
            tUs[e] = (b[4] << 16) | (b[5] << 8) | b[6];
        }
    }
}

/* tensor is [C][H][W][T]; base holds the values from before the call (may be tensor itself for
 * mode 0 = OR; for mode 1 = SUM it must be an untouched copy). */
void oracle_bin_events_f32(float *tensor, const float *base, const int32_t *x, const int32_t *y,
                           const int32_t *p, const double *tMs, int64_t nEvents, int64_t timeShift,
                           int32_t C, int32_t H, int32_t W, int32_t T, double samplingTime, int32_t mode)
{
    const float value = (float)(1.0 / samplingTime);
    for (int64_t e = 0; e < nEvents; ++e) {
        const double bin = rint(tMs[e] / samplingTime) - (double)timeShift;
        const int32_t ye = y ? y[e] : 0;
        if (!(bin >= 0.0 && bin < (double)T)) continue;
        if (x[e] < 0 || x[e] >= W || ye < 0 || ye >= H || p[e] < 0 || p[e] >= C) continue;
        const int64_t idx = (((int64_t)p[e] * H + ye) * W + x[e]) * T + (int64_t)bin;
        tensor[idx] = mode == 0 ? value : base[idx] + value;
    }
}

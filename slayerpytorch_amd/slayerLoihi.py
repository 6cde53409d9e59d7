"""Host side of the Loihi hot path: the part of the reference's ``slayerLoihi.spikeLayer``
that feeds and wraps the Loihi neuron kernel, re-hosted on PyTorch-ROCm.

Mirrors: threshold ``theta = vThMant * 2**6`` (src/slayerLoihi.py:47-56), the integer PSP and
refractory kernel generators (:58-89), ``spikeLoihi`` / ``spikeLoihiFull`` (:91-122), the
autograd Function ``_spike`` (:243-283) and the quantised ``dense`` default (:124-139,
src/quantizeParams.py).
"""
import numpy as np
import torch

from . import slayer, slayerCuda, slayerLoihiCuda


class quantizeWeights(torch.autograd.Function):
    """``round(w / step) * step`` with a straight-through gradient (src/quantizeParams.py:3-31)."""

    @staticmethod
    def forward(ctx, weights, step=1):
        if weights.is_cuda and weights.dtype == torch.float32 and weights.is_contiguous() and weights.numel() > 0 \
                and not isinstance(step, torch.Tensor):
            return slayerLoihiCuda.quantize(weights, float(step))   # the same values from one kernel
        return torch.round(weights / step) * step

    @staticmethod
    def backward(ctx, gradOutput):
        return gradOutput, None


def quantize(weights, step=1):
    return quantizeWeights.apply(weights, step)


def loihiPspKernel(iDecay, vDecay, wgtExp=0):
    """Voltage response of the CUBA neuron to one input spike of weight 1, as a float list:
    integer recurrence started at ``1 << (7 + wgtExp)`` (a weight of 2), run until the voltage
    reaches zero (the final 0 is kept) and halved (src/slayerLoihi.py:66-79)."""
    u = [1 << (6 + wgtExp + 1)]
    v = [u[-1]]
    while v[-1] > 0:
        uNext = (u[-1] * ((1 << 12) - iDecay)) >> 12
        vNext = ((v[-1] * ((1 << 12) - vDecay)) >> 12) + uNext
        u.append(uNext)
        v.append(vNext)
    return [float(x) / 2 for x in v]


def loihiRefKernel(theta, vDecay, refDelay, SCALE=1000):
    """Absolute refractory block (``refDelay`` samples of ``-SCALE*theta``, first one 0) followed
    by ``-2 *`` the decaying threshold sequence (src/slayerLoihi.py:81-89)."""
    absolute = np.ones(refDelay) * (-SCALE * theta)
    absolute[0] = 0
    relative = [theta]
    while relative[-1] > 0:
        relative.append((relative[-1] * ((1 << 12) - vDecay)) >> 12)
    return np.concatenate((absolute, -2 * np.array(relative))).astype("float32")


class spikeLayer(slayer.spikeLayer):
    """Loihi flavour of :class:`slayer.spikeLayer`.  ``neuronDesc`` needs ``vThMant, vDecay,
    iDecay, refDelay, wgtExp, tauRho, scaleRho``; ``theta`` is derived and ``scaleRho`` is
    divided by the PSP kernel's maximum, both written back into ``neuronDesc`` as the
    reference does."""

    def __init__(self, neuronDesc, simulationDesc):
        if neuronDesc["type"] == "LOIHI":
            neuronDesc["theta"] = neuronDesc["vThMant"] * 2 ** 6
        super().__init__(neuronDesc, simulationDesc)
        self.maxPspKernel = torch.max(self.srmKernel).cpu().data.item()
        neuronDesc["scaleRho"] /= self.maxPspKernel

    def calculateSrmKernel(self):
        return torch.tensor(loihiPspKernel(self.neuron["iDecay"], self.neuron["vDecay"], self.neuron["wgtExp"]))

    def calculateRefKernel(self, SCALE=1000):
        return torch.tensor(loihiRefKernel(self.neuron["theta"], self.neuron["vDecay"],
                                           self.neuron["refDelay"], SCALE))

    def spikeLoihi(self, weightedSpikes, delay=0, delayTs=1):
        """Loihi neuron dynamics on weighted (unfiltered) input spikes -> output spikes, with the
        SLAYER surrogate gradient attached.  ``delay`` (extension) gives
        ``delayShift(spikeLoihi(x), delay, delayTs)`` - a shift by ``int(delay / delayTs)`` samples
        - from the same kernel."""
        Ts = self.simulation["Ts"]
        scalar = not isinstance(delay, torch.Tensor) and not isinstance(delayTs, torch.Tensor) and np.ndim(delay) == 0
        if scalar:
            # the shift kernel's own arithmetic: the fp32 quotient, truncated toward zero
            quotient = np.float32(delay) / np.float32(delayTs)
            steps = int(quotient) if np.isfinite(quotient) else -1
            if 0 <= steps <= slayerLoihiCuda.MAX_FUSED_DELAY:
                return _spike.apply(weightedSpikes, self.srmKernel, self.neuron, Ts, steps)
        # a delay per neuron, a tensor, a negative or a long delay: the separate shift
        return self.delayShift(_spike.apply(weightedSpikes, self.srmKernel, self.neuron, Ts, 0), delay, delayTs)

    def spikeLoihiFull(self, weightedSpikes):
        """Same dynamics without autograd; returns ``(spike, voltage, current)``."""
        return _spike.loihi(weightedSpikes, self.neuron, self.simulation["Ts"])

    def dense(self, inFeatures, outFeatures, weightScale=100, preHookFx=lambda x: quantize(x, step=2)):
        return super().dense(inFeatures, outFeatures, weightScale, preHookFx)

    def conv(self, inChannels, outChannels, kernelSize, stride=1, padding=0, dilation=1, groups=1, weightScale=100,
             preHookFx=lambda x: quantize(x, step=2)):
        """Convolution synapse with weights quantised in steps of 2 (src/slayerLoihi.py:141-156)."""
        return super().conv(inChannels, outChannels, kernelSize, stride, padding, dilation, groups, weightScale,
                            preHookFx)

    def _poolWeight(self):
        # the pooling weight that makes one input spike cross the threshold, on Loihi's even weight grid
        # (src/slayerLoihi.py:171-174); the layer multiplies its argument by 1.1 again
        return float(quantize(torch.tensor(1.1 * self.neuron["theta"] / self.maxPspKernel), 2)) / 1.1

    def pool(self, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        """Pooling synapse (src/slayerLoihi.py:158-174)."""
        return slayer._poolLayer(self._poolWeight(), kernelSize, stride, padding, dilation, preHookFx)

    def convTranspose(self, inChannels, outChannels, kernelSize, stride=1, padding=0, dilation=1, groups=1,
                      weightScale=100, preHookFx=lambda x: quantize(x, step=2)):
        """Transposed convolution synapse with quantised weights (src/slayerLoihi.py:175-189)."""
        return super().convTranspose(inChannels, outChannels, kernelSize, stride, padding, dilation, groups,
                                     weightScale, preHookFx)

    def unpool(self, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        """Unpooling synapse (src/slayerLoihi.py:191-205)."""
        return slayer._unpoolLayer(self._poolWeight(), kernelSize, stride, padding, dilation, preHookFx)


class _spike(torch.autograd.Function):
    @staticmethod
    def _scaled(weightedSpikes, Ts):
        # the reference multiplies by Ts unconditionally; by 1 that is a copy of the tensor
        if weightedSpikes.dtype == torch.int32:
            Ts = 1
        x = weightedSpikes if Ts == 1 else weightedSpikes * Ts
        return x.contiguous(), Ts

    @staticmethod
    def loihi(weightedSpikes, neuron, Ts):
        x, Ts = _spike._scaled(weightedSpikes, Ts)
        spike, voltage, current = slayerLoihiCuda.getSpikes(
            x, neuron["wgtExp"], neuron["theta"], neuron["iDecay"], neuron["vDecay"], neuron["refDelay"])
        return (spike if Ts == 1 else spike / Ts), voltage, current

    @staticmethod
    def forward(ctx, weightedSpikes, srmKernel, neuron, Ts, delaySteps=0):
        # the layer needs the voltage for the backward pass only, and never the current
        needVoltage = ctx.needs_input_grad[0]
        x, scale = _spike._scaled(weightedSpikes, Ts)
        spike, voltage, _ = slayerLoihiCuda.getSpikesDelayed(
            x, neuron["wgtExp"], neuron["theta"], neuron["iDecay"], neuron["vDecay"], neuron["refDelay"],
            delaySteps, voltage=needVoltage, current=False)
        if scale != 1:
            spike = spike / scale
        if needVoltage:
            ctx.save_for_backward(voltage, srmKernel.clone().detach())
        ctx.theta = float(neuron["theta"])
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        ctx.Ts = float(Ts)
        ctx.delaySteps = int(delaySteps)
        return spike

    @staticmethod
    def backward(ctx, gradOutput):
        voltage, srmKernel = ctx.saved_tensors
        gradOutput = gradOutput.contiguous()
        if ctx.delaySteps:   # adjoint of the fused delay: the gradient moves back by as many samples
            gradOutput = slayerCuda.shift(gradOutput, float(ctx.delaySteps), 1.0, sign=-1.0)
        # surrogate gradient and correlation with the PSP kernel in one kernel
        return slayerCuda.spikeBackwardCorr(gradOutput, voltage, srmKernel, ctx.theta,
                                            ctx.pdfTimeConstant, ctx.pdfScale, ctx.Ts), None, None, None, None

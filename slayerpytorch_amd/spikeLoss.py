"""Spike-train losses on top of the PSP kernel (src/spikeLoss.py:7-104), computed on the device.

``spikeTime``: half the squared van Rossum distance between output and desired spike trains, from the
fused error + squared-sum kernels of ``slayerCuda.spikeLoss`` (rows too long for them take the tensor
expression of the reference).
``numSpikes``: spike count inside a target region against a desired count, spike-time loss
outside it.  The reference builds the target region, the desired counts and the count error on
the host (numpy round trips, src/spikeLoss.py:91-102); here every step is a tensor operation on
the device of ``spikeOut``, so the loss never synchronises with the host.
"""
import torch

from . import slayerCuda
from .slayer import spikeLayer


class _spikeLossFunction(torch.autograd.Function):
    """``1/2 * sum((psp(out - desired) + addend)**2) * Ts`` over ``slayerCuda.spikeLoss``; the backward
    pass is the correlation of the saved error signal, as autograd derives it for the reference's
    expression (src/spikeLoss.py:56-58)."""

    @staticmethod
    def forward(ctx, spikeOut, spikeDesired, addend, srmKernel, Ts):
        result = slayerCuda.spikeLoss(spikeOut.contiguous(), spikeDesired.contiguous(), srmKernel, Ts,
                                      None if addend is None else addend.contiguous())
        loss, error = result
        ctx.save_for_backward(error, srmKernel)
        ctx.Ts = float(Ts)
        return loss

    @staticmethod
    def backward(ctx, gradLoss):
        error, srmKernel = ctx.saved_tensors
        grad = slayerCuda.corr(error * (gradLoss * ctx.Ts), srmKernel, ctx.Ts)
        return (grad if ctx.needs_input_grad[0] else None, -grad if ctx.needs_input_grad[1] else None,
                None, None, None)


def _fits(spike, srmKernel):
    # the fused loss keeps one row and the filter in the LDS of a work-group
    return spike.is_cuda and spike.dtype == torch.float32 and (spike.shape[-1] + 2 * srmKernel.numel()) * 4 <= 60 * 1024


class spikeLoss(torch.nn.Module):
    """``spikeLoss(networkDescriptor, slayerClass=spikeLayer)`` with ``networkDescriptor`` holding
    ``neuron``, ``simulation`` and ``training.error`` (``type`` and, for ``NumSpikes``,
    ``tgtSpikeRegion`` {start, stop} and ``tgtSpikeCount`` {True, False})."""

    def __init__(self, networkDescriptor, slayerClass=spikeLayer):
        super().__init__()
        self.neuron = networkDescriptor["neuron"]
        self.simulation = networkDescriptor["simulation"]
        self.errorDescriptor = networkDescriptor["training"]["error"]
        self.slayer = slayerClass(self.neuron, self.simulation)

    def spikeTime(self, spikeOut, spikeDesired):
        """``1/2 * sum(psp(spikeOut - spikeDesired)^2) * Ts`` (src/spikeLoss.py:37-58)."""
        assert self.errorDescriptor["type"] == "SpikeTime", "Error type is not SpikeTime"
        Ts = self.simulation["Ts"]
        if _fits(spikeOut, self.slayer.srmKernel):
            return _spikeLossFunction.apply(spikeOut, spikeDesired, None, self.slayer.srmKernel, Ts)
        error = self.slayer.psp(spikeOut - spikeDesired)
        return 1 / 2 * torch.sum(error ** 2) * Ts

    def numSpikes(self, spikeOut, desiredClass, numSpikesScale=1):
        """Spike-count loss (src/spikeLoss.py:60-104).  ``desiredClass`` is one-hot with a time
        dimension of 1.  Inside the target region the error is ``(actual - desired spike count)
        / region length * numSpikesScale`` (a constant, no gradient, as in the reference);
        outside it every output spike is penalised through the PSP kernel."""
        assert self.errorDescriptor["type"] == "NumSpikes", "Error type is not NumSpikes"
        Ts = self.simulation["Ts"]
        region = self.errorDescriptor["tgtSpikeRegion"]
        count = self.errorDescriptor["tgtSpikeCount"]
        startID = int(round(region["start"] / Ts))      # round half to even, like numpy.rint
        stopID = int(round(region["stop"] / Ts))
        with torch.no_grad():
            out = spikeOut.detach()
            inRegion = torch.zeros(out.shape[-1], dtype=out.dtype, device=out.device)
            inRegion[startID:stopID] = 1
            actualSpikes = torch.sum(out[..., startID:stopID], 4, keepdim=True) * Ts
            # the count error in double precision, rounded to fp32 at the end, as the reference's numpy does
            desiredSpikes = torch.where(desiredClass.to(out.device) == True,            # noqa: E712
                                        torch.as_tensor(float(count[True]), dtype=torch.float64, device=out.device),
                                        torch.as_tensor(float(count[False]), dtype=torch.float64, device=out.device))
            errorSpikeCount = (actualSpikes.double() - desiredSpikes) / (stopID - startID) * numSpikesScale
            spikeDesired = out * inRegion                 # the output's own spikes inside the region
            countError = (errorSpikeCount * inRegion.double()).to(out.dtype)
        if _fits(spikeOut, self.slayer.srmKernel):
            return _spikeLossFunction.apply(spikeOut, spikeDesired, countError, self.slayer.srmKernel, Ts)
        error = self.slayer.psp(spikeOut - spikeDesired)
        error = error + countError
        return 1 / 2 * torch.sum(error ** 2) * Ts

"""Spike-train losses on top of the PSP kernel (src/spikeLoss.py:7-104), computed on the device.

``spikeTime``: half the squared van Rossum distance between output and desired spike trains.
``numSpikes``: spike count inside a target region against a desired count, spike-time loss
outside it.  The reference builds the target region, the desired counts and the count error on
the host (numpy round trips, src/spikeLoss.py:91-102); here every step is a tensor operation on
the device of ``spikeOut``, so the loss never synchronises with the host.
"""
import torch

from .slayer import spikeLayer


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
        error = self.slayer.psp(spikeOut - spikeDesired)
        return 1 / 2 * torch.sum(error ** 2) * self.simulation["Ts"]

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
        error = self.slayer.psp(spikeOut - spikeDesired)
        error = error + countError
        return 1 / 2 * torch.sum(error ** 2) * Ts

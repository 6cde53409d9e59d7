"""Host side of the SRM hot path: the part of the reference's ``slayer.spikeLayer`` that feeds
and wraps the temporal kernels, re-hosted on PyTorch-ROCm.

Mirrors, with the same names, signatures and side effects:

* kernel generators ``calculateSrmKernel`` / ``calculateRefKernel`` / ``_calculateAlphaKernel``
  (src/slayer.py:98-123),
* ``spikeLayer.psp`` / ``spike`` / ``delayShift`` / ``delay`` (src/slayer.py:130-142, 333-391),
* autograd Functions ``_spikeFunction``, ``_pspFunction``, ``_delayLayer``, ``_delayFunction``,
  ``_delayFunctionNoGradient`` (src/slayer.py:817-979),
* ``dense`` (src/slayer.py:144-172, 393-437) as one library GEMM per batch item,
* ``conv`` / ``pool`` / ``convTranspose`` / ``unpool`` (src/slayer.py:207-312, 451-748) over the
  per-timestep synapse kernels of :mod:`slayerpytorch_amd.synapse` instead of ``F.conv3d`` /
  ``F.conv_transpose3d`` with a (KH, KW, 1) kernel.

Differences from the reference, all on the host: backward passes use the fused
``slayerCuda.spikeBackward`` / ``slayerCuda.delayGrad`` kernels instead of chains of
elementwise torch ops, and scalars saved for backward stay Python floats (no 0-dim device
tensors, hence no device-to-host synchronisation in backward).
"""
import math
import weakref

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F
from torch.utils.weak import WeakTensorKeyDictionary

from . import slayerCuda
from . import synapse


# spikeLayer.psp filters with the alpha kernel as a recursion over time when the kernel has more taps than this
# (shorter kernels are memory streams as sums already); PSP_RECURSION = False keeps the sums everywhere.
PSP_RECURSION = True
PSP_RECURSION_MIN_TAPS = 16


def alphaKernel(tau, Ts, tSample, mult=1.0, EPSILON=0.01):
    """Samples ``mult * t/tau * exp(1 - t/tau)`` at t = 0, Ts, 2Ts, ... < tSample and stops
    (exclusively) at the first sample past the peak whose magnitude is below ``EPSILON``
    (src/slayer.py:114-123).  Evaluated in float64; returns a Python list."""
    values = []
    for t in np.arange(0, tSample, Ts):
        v = mult * t / tau * math.exp(1 - t / tau)
        if abs(v) < EPSILON and t > tau:
            break
        values.append(v)
    return values


class spikeLayer(nn.Module):
    """SRM spiking layer engine: PSP filter, spike function and delays on NCHWT tensors.

    ``neuronDesc`` needs ``theta, tauSr, tauRef, scaleRef, tauRho, scaleRho``; ``simulationDesc``
    needs ``Ts, tSample`` (src/slayer.py:47-96).
    """

    def __init__(self, neuronDesc, simulationDesc, fullRefKernel=False):
        super().__init__()
        self.neuron = neuronDesc
        self.simulation = simulationDesc
        self.fullRefKernel = fullRefKernel
        self.register_buffer("srmKernel", self.calculateSrmKernel())
        self.register_buffer("refKernel", self.calculateRefKernel())

    def calculateSrmKernel(self):
        return torch.FloatTensor(self._calculateAlphaKernel(self.neuron["tauSr"]))

    def calculateRefKernel(self):
        mult = -self.neuron["scaleRef"] * self.neuron["theta"]
        if self.fullRefKernel:
            kernel = self._calculateAlphaKernel(tau=self.neuron["tauRef"], mult=mult, EPSILON=0.0001)
        else:
            kernel = self._calculateAlphaKernel(tau=self.neuron["tauRef"], mult=mult)
        return torch.FloatTensor(kernel)

    def _calculateAlphaKernel(self, tau, mult=1, EPSILON=0.01):
        return alphaKernel(tau, self.simulation["Ts"], self.simulation["tSample"], mult, EPSILON)

    def psp(self, spike):
        """PSP filtering of a spike tensor (same shape out).  While ``srmKernel`` is the alpha kernel
        that ``calculateSrmKernel`` built (checked once per kernel tensor, against the values
        computed on the host) and has more than ``PSP_RECURSION_MIN_TAPS`` taps, filter and
        gradient run as a recursion over time (``slayerCuda.pspAlpha``), which agrees with the
        sum over the taps to rounding; a kernel that was replaced or edited takes the sums."""
        alpha = self._srmKernelIsAlpha()
        origin = _fresh_spikes(spike) if alpha is not None and _recursion_serves(spike) else None
        if origin is not None:
            return _pspOfSpikeFunction.apply(spike, origin[0], self.srmKernel, self.simulation["Ts"], alpha, *origin[1:])
        psp = _pspFunction.apply(spike, self.srmKernel, self.simulation["Ts"], alpha)
        if PAIR_SPIKE_PSP and alpha is not None and psp.requires_grad and _recursion_serves(spike):
            # for spike(): what this signal was filtered from, and that it has not been touched since
            _pspNotes[psp] = (spike, self.srmKernel, alpha, psp._version)
        return psp

    def _srmKernelIsAlpha(self):
        """(tau, mult) when ``srmKernel`` still holds ``alphaKernel(tauSr, ...)`` and the recursion
        is switched on, else None.  Comparing costs a copy to the host, so the verdict is kept per
        tensor object and version."""
        kernel = self.srmKernel
        if not PSP_RECURSION or not kernel.is_cuda or kernel.numel() <= PSP_RECURSION_MIN_TAPS:
            return None
        stamp = (id(kernel), kernel.data_ptr(), kernel._version)
        if getattr(self, "_srmAlphaStamp", None) != stamp:
            tau = self.neuron.get("tauSr") if hasattr(self.neuron, "get") else None   # (the Loihi layer has none)
            same = False
            if tau is not None and float(tau) > 0:
                expected = torch.FloatTensor(self._calculateAlphaKernel(tau))
                same = kernel.shape == expected.shape and kernel.dtype == expected.dtype and \
                    bool(torch.equal(kernel.detach().cpu(), expected))
            self._srmAlphaStamp = stamp
            self._srmAlpha = (float(tau), 1.0) if same else None
        return self._srmAlpha

    def spike(self, membranePotential):
        """Spike function with refractory response.  A contiguous ``membranePotential`` is
        updated in place with the refractory response, as in the reference."""
        origin = _pspNotes.pop(membranePotential, None) if PAIR_SPIKE_PSP else None   # (the note is what keeps x alive)
        if origin is not None and torch.is_grad_enabled() and membranePotential.requires_grad \
                and membranePotential.is_contiguous() and membranePotential._version == origin[3] \
                and isinstance(membranePotential.grad_fn, _pspFunction._backward_cls) \
                and _unobserved(membranePotential) and origin[0].shape == membranePotential.shape:
            # spike(psp(x)), the ordering of the reference's MLP example: the spikes' gradient goes past the PSP
            # filter straight to x, surrogate gradient and correlation in one kernel
            return _spikeOfPspFunction.apply(membranePotential, origin[0], self.refKernel, origin[1], self.neuron,
                                             self.simulation["Ts"], origin[2])
        spikes = _spikeFunction.apply(membranePotential, self.refKernel, self.neuron, self.simulation["Ts"])
        if PAIR_SPIKE_PSP and spikes.requires_grad:
            # for psp(): which potential these spikes came from (kept alive by the spike function's own record for the
            # backward pass, not by this note), and that neither has been touched since
            _spikeNotes[spikes] = (weakref.ref(membranePotential), float(self.neuron["theta"]),
                                   float(self.neuron["tauRho"] * self.neuron["theta"]), float(self.neuron["scaleRho"]),
                                   spikes._version, membranePotential._version)
        return spikes

    def spikeDelayed(self, membranePotential, delay, Ts=None):
        """``delayShift(spike(membranePotential), delay, Ts)`` or, with a ``_delayLayer`` as ``delay``,
        ``delay(spike(membranePotential))`` (src/slayer.py:333-391) from one kernel: the spikes are
        shifted while they are stored, and the backward pass shifts the gradient while it applies the
        surrogate gradient.  A delay layer's delays receive their gradient as in the reference."""
        Ts = self.simulation["Ts"] if Ts is None else Ts
        if isinstance(delay, _delayLayer):
            N, C, H, W, Ns = membranePotential.shape
            table = delay.delay
            if membranePotential.numel() != table.numel() * Ns * N:
                table = table.repeat((1, H, W))
            return _spikeDelayedFunction.apply(membranePotential, self.refKernel, self.neuron, self.simulation["Ts"],
                                               table, delay.Ts)
        return _spikeDelayedFunction.apply(membranePotential, self.refKernel, self.neuron, self.simulation["Ts"],
                                           delay, Ts)

    def pspSpike(self, input):
        """``spike(psp(input))`` - the layer ordering of the reference's MLP example
        (example/02_NMNIST_MLP/nmnistMLP.py:59-60) - as one Function with one backward kernel
        (extension; same values as the two calls)."""
        return _pspSpikeFunction.apply(input, self.srmKernel, self.refKernel, self.neuron, self.simulation["Ts"],
                                       self._srmKernelIsAlpha())

    def spikePsp(self, membranePotential):
        """``s = spike(membranePotential)`` and ``psp(s)``, returned as the pair ``(s, psp(s))`` - what every layer
        of the reference's convolutional example does with its spikes, ``spike(conv(psp(spike(...))))``
        (example/03_NMNIST_CNN/nmnistCNN.py:55-60) - as one Function whose backward pass is one kernel
        (extension; same values as the two calls, gradients to rounding)."""
        return _spikePspFunction.apply(membranePotential, self.refKernel, self.srmKernel, self.neuron,
                                       self.simulation["Ts"], self._srmKernelIsAlpha())

    def delayShift(self, input, delay, Ts=1):
        """Delays ``input`` in time by ``delay`` (number, one-element tensor, or one value per
        neuron); the gradient flows to ``input`` only."""
        origin = _fresh_spikes(input) if isinstance(input, torch.Tensor) and input.dim() == 5 else None
        if origin is not None:
            return _delayOfSpikeFunction.apply(input, origin[0], delay, Ts, False, *origin[1:])
        return _delayFunctionNoGradient.apply(input, delay, Ts)

    def delay(self, inputSize):
        """Learnable per-neuron (or per-channel) delay module for inputs of spatial shape
        ``inputSize`` = C or (C, H, W)."""
        return _delayLayer(inputSize, self.simulation["Ts"])

    def dense(self, inFeatures, outFeatures, weightScale=10, preHookFx=None):
        """Fully connected synapse applied per time step."""
        return _denseLayer(inFeatures, outFeatures, weightScale, preHookFx)

    def conv(self, inChannels, outChannels, kernelSize, stride=1, padding=0, dilation=1, groups=1,
             weightScale=100, preHookFx=None):
        """Convolution synapse over (H, W), applied per time step (src/slayer.py:207-234)."""
        return _convLayer(inChannels, outChannels, kernelSize, stride, padding, dilation, groups, weightScale,
                          preHookFx)

    def pool(self, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        """Sum-pooling synapse with weights ``1.1 * theta`` (src/slayer.py:236-259)."""
        return _poolLayer(self.neuron["theta"], kernelSize, stride, padding, dilation, preHookFx)

    def convTranspose(self, inChannels, outChannels, kernelSize, stride=1, padding=0, dilation=1, groups=1,
                      weightScale=100, preHookFx=None):
        """Transposed convolution synapse (src/slayer.py:261-288)."""
        return _convTransposeLayer(inChannels, outChannels, kernelSize, stride, padding, dilation, groups,
                                   weightScale, preHookFx)

    def unpool(self, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        """Unpooling synapse with weights ``1.1 * theta`` (src/slayer.py:290-313)."""
        return _unpoolLayer(self.neuron["theta"], kernelSize, stride, padding, dilation, preHookFx)

    def dropout(self, p=0.5, inplace=False):
        """Dropout that keeps a dropped neuron dropped for the whole time axis (src/slayer.py:315-331);
        a plain PyTorch module, as in the reference."""
        return _dropoutLayer(p, inplace)

    def replicateInTime(self, input, mode="nearest"):
        """Repeats an (N, C, H, W) tensor along a new time axis of tSample / Ts samples
        (src/slayer.py:179-185)."""
        Ns = int(self.simulation["tSample"] / self.simulation["Ts"])
        N, C, H, W = input.shape
        if mode != "nearest":
            raise Exception("Unsupported mode. It was {}".format(mode))
        return F.interpolate(input.reshape(N, C, H, W, 1), size=(H, W, Ns), mode="nearest")


# psp(s) of a tensor s that spike() has just returned - what the layers of the reference's convolutional example
# do, spike(conv(psp(spike(...)))) - sends its gradient past the spike function straight to the membrane
# potential: correlation and surrogate gradient in one kernel (slayerCuda.pspSpikeBackwardAlpha) instead of
# two with a tensor in between.  Gradients that reach s from elsewhere still pass through the spike function's
# own backward pass; the sum at the membrane potential is the same.  Likewise spike(u) of a signal u that psp() has
# just returned - the ordering of the reference's MLP example, spike(psp(fc(x))) - sends the spikes' gradient past
# the PSP filter (slayerCuda.spikeBackwardPspAlpha), and delay(s) / delayShift(s, d) of fresh spikes sends its gradient
# past the spike function as well (slayerCuda.spikeBackwardDelayed).  False keeps the Functions apart.
PAIR_SPIKE_PSP = True


# The dense layer's product and weight gradient event by event (synapse.denseEvents, denseEventsGradWeight)
# when its input is sparse enough and has enough channels for that to pay: True / False force the choice,
# "auto" counts the non-zero inputs of a layer on the device - at its first two calls, whenever the input's shape
# changes and at every DENSE_EVENTS_CHECK_EVERY-th call - and copies the count to pinned host memory without
# waiting for it: a call uses the latest count that has arrived (at most a few calls old), and only a layer's very
# first call waits.  Nothing is measured while a HIP graph is being captured: the last count decides then.
DENSE_EVENTS = "auto"
DENSE_EVENTS_MAX_DENSITY = 0.05           # weight gradient
DENSE_EVENTS_MAX_DENSITY_FORWARD = 0.03   # product (its input has to be transposed first)
DENSE_EVENTS_MIN_CHANNELS = 1024
DENSE_EVENTS_CHECK_EVERY = 4

# The dense layer's product and input gradient from synapse.denseRows where that pays (layers with up to 448 inputs).
# False keeps the library products.
DENSE_ROWS = True


class _denseLayer(nn.Conv3d):
    """Fully connected synapse: an (outFeatures, C, H, W, 1) weight applied at every time step
    (src/slayer.py:393-440)."""

    def __init__(self, inFeatures, outFeatures, weightScale=1, preHookFx=None):
        if isinstance(inFeatures, int):
            kernel, inChannels = (1, 1, 1), inFeatures
        elif len(inFeatures) == 2:
            kernel, inChannels = (inFeatures[1], inFeatures[0], 1), 1
        elif len(inFeatures) == 3:
            kernel, inChannels = (inFeatures[1], inFeatures[0], 1), inFeatures[2]
        else:
            raise Exception("inFeatures should not be more than 3 dimension. It was: {}".format(inFeatures))
        if not isinstance(outFeatures, int):
            raise Exception("outFeatures should not be more than 1 dimesnion. It was: {}".format(outFeatures))
        super().__init__(inChannels, outFeatures, kernel, bias=False)
        if weightScale != 1:
            self.weight = nn.Parameter(weightScale * self.weight)
        self.preHookFx = preHookFx
        self._eventCalls = 0
        self._eventDensity = None     # latest fraction of non-zero inputs that has arrived on the host
        self._eventShape = None
        self._eventPending = None     # (pinned host count, event recorded after its copy, numel)

    def _measureDensity(self, x):
        """Keeps ``_eventDensity`` current without stalling the stream (see DENSE_EVENTS)."""
        shape = tuple(x.shape)
        if shape != self._eventShape:
            self._eventShape, self._eventCalls, self._eventDensity, self._eventPending = shape, 0, None, None
        if self._eventPending is not None and self._eventPending[1].query():
            self._eventDensity = int(self._eventPending[0]) / self._eventPending[2]
            self._eventPending = None
        if self._eventPending is None and (self._eventCalls < 2 or self._eventCalls % DENSE_EVENTS_CHECK_EVERY == 0):
            count = torch.empty((), dtype=torch.int64, pin_memory=True)
            count.copy_(torch.count_nonzero(x), non_blocking=True)
            arrived = torch.cuda.Event()
            arrived.record()
            self._eventPending = (count, arrived, x.numel())
            if self._eventDensity is None:      # the first call of this shape has nothing older to go by
                arrived.synchronize()
                self._eventDensity, self._eventPending = int(count) / x.numel(), None
        self._eventCalls += 1

    def _inputIsSparse(self, x):
        """(product, weight gradient): which of the two are summed over the events in this call (see DENSE_EVENTS)."""
        N, K, T = x.shape
        if DENSE_EVENTS is False or not x.is_cuda or x.dtype != torch.float32 or x.numel() == 0 \
                or not synapse.denseEventsSupported(N, K, self.weight.shape[0], T):
            return False, False
        if DENSE_EVENTS is True:
            return True, True
        if K < DENSE_EVENTS_MIN_CHANNELS:
            return False, False
        if not torch.cuda.is_current_stream_capturing():
            self._measureDensity(x)
        if self._eventDensity is None:
            return False, False
        return self._eventDensity <= DENSE_EVENTS_MAX_DENSITY_FORWARD, self._eventDensity <= DENSE_EVENTS_MAX_DENSITY

    def forward(self, input):
        weight = self.weight if self.preHookFx is None else self.preHookFx(self.weight)
        # The kernel spans the whole (H, W) extent of the input, so the layer is one matrix product
        # per batch item, W[O, C*H*W] x X[C*H*W, T], with time innermost as the tensor already is:
        # a plain library GEMM instead of a 3-D convolution with a degenerate kernel; for the spike
        # tensors these layers usually see, product and weight gradient are sums over the events instead.
        if input.dim() == 5 and tuple(input.shape[1:4]) == tuple(weight.shape[1:4]) and self.bias is None:
            N, T = input.shape[0], input.shape[4]
            O, K = weight.shape[0], weight.shape[1] * weight.shape[2] * weight.shape[3]
            product, gradient = self._inputIsSparse(input.reshape(N, K, T))
            if product or gradient:
                return synapse.synapseDenseEvents(input.reshape(N, K, T), weight.reshape(O, K), product,
                                                  gradient).reshape(N, O, 1, 1, T)
            # layers with few inputs: the library spends its time on fp32 matrix instructions; one kernel with the
            # weights in registers and bf16 instructions over split operands is 1.5 to 2.5 times as fast
            if DENSE_ROWS and input.is_cuda and input.dtype == torch.float32 and weight.dtype == torch.float32 \
                    and synapse.denseRowsPays(N, K, O, T):
                return synapse.synapseDenseRows(input.reshape(N, K, T), weight.reshape(O, K)).reshape(N, O, 1, 1, T)
            # batched product with the weight matrix repeated by a zero stride: torch.matmul of a
            # 2-D by a 3-D tensor would first copy the input into a (K, N*T) layout
            return torch.bmm(weight.reshape(1, O, K).expand(N, O, K), input.reshape(N, K, T)).reshape(N, O, 1, 1, T)
        return F.conv3d(input, weight, self.bias, self.stride, self.padding, self.dilation, self.groups)


def _hw(value, name, default=None):
    """An int or a pair as the (h, w, time) triple torch's 3-D modules take, the way the reference's
    layers expand their arguments (src/slayer.py:456-487)."""
    if value is None:
        return default
    if isinstance(value, int):
        return (value, value, 1 if name != "padding" else 0)
    if len(value) == 2:
        return (value[0], value[1], 1 if name != "padding" else 0)
    raise Exception("{} can be either int or tuple of size 2. It was: {}".format(name, value))


class _convLayer(nn.Conv3d):
    """Convolution synapse (src/slayer.py:451-507): a (outFeatures, inFeatures/groups, KH, KW, 1)
    weight applied at every time step by the per-timestep synapse kernel."""

    def __init__(self, inFeatures, outFeatures, kernelSize, stride=1, padding=0, dilation=1, groups=1,
                 weightScale=1, preHookFx=None):
        super().__init__(inFeatures, outFeatures, _hw(kernelSize, "kernelSize"), _hw(stride, "stride"),
                         _hw(padding, "padding"), _hw(dilation, "dilation"), groups, bias=False)
        if weightScale != 1:
            self.weight = nn.Parameter(weightScale * self.weight)
        self.preHookFx = preHookFx

    def forward(self, input):
        weight = self.weight if self.preHookFx is None else self.preHookFx(self.weight)
        return synapse.synapseConv(input, weight, self.stride[:2], self.padding[:2], self.dilation[:2],
                                   self.groups)


def _poolWeight(theta, shape):
    return nn.Parameter(torch.full(shape, 1.1 * theta, dtype=torch.float32), requires_grad=False)


class _poolLayer(nn.Conv3d):
    """Sum pooling as a 1 -> 1 channel synapse with constant weights ``1.1 * theta`` on the tensor
    viewed as (N, 1, C*H, W, T) (src/slayer.py:509-577).  Like the reference, an extent that is not
    a multiple of the window is extended by ``extent % window`` rows of zeros."""

    def __init__(self, theta, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        kernel = _hw(kernelSize, "kernelSize")
        super().__init__(1, 1, kernel, _hw(stride, "stride", kernel), _hw(padding, "padding"),
                         _hw(dilation, "dilation"), bias=False)
        self.weight = _poolWeight(theta, self.weight.shape)
        self.preHookFx = preHookFx

    def forward(self, input):
        kH, kW = self.weight.shape[2], self.weight.shape[3]
        if input.shape[2] % kH != 0:
            input = torch.cat((input, input.new_zeros((input.shape[0], input.shape[1], input.shape[2] % kH,
                                                       input.shape[3], input.shape[4]))), 2)
        if input.shape[3] % kW != 0:
            input = torch.cat((input, input.new_zeros((input.shape[0], input.shape[1], input.shape[2],
                                                       input.shape[3] % kW, input.shape[4]))), 3)
        N, C, H, W, T = input.shape
        weight = self.weight if self.preHookFx is None else self.preHookFx(self.weight)
        result = synapse.synapseConv(input.reshape(N, 1, C * H, W, T), weight, self.stride[:2], self.padding[:2],
                                     self.dilation[:2], 1)
        return result.reshape(result.shape[0], C, -1, result.shape[3], result.shape[4])


class _convTransposeLayer(nn.ConvTranspose3d):
    """Transposed convolution synapse (src/slayer.py:579-643)."""

    def __init__(self, inFeatures, outFeatures, kernelSize, stride=1, padding=0, dilation=1, groups=1,
                 weightScale=1, preHookFx=None):
        super().__init__(inFeatures, outFeatures, _hw(kernelSize, "kernelSize"), _hw(stride, "stride"),
                         _hw(padding, "padding"), 0, groups, False, _hw(dilation, "dilation"))
        if weightScale != 1:
            self.weight = nn.Parameter(weightScale * self.weight)
        self.preHookFx = preHookFx

    def forward(self, input):
        weight = self.weight if self.preHookFx is None else self.preHookFx(self.weight)
        return synapse.synapseConvTranspose(input, weight, self.stride[:2], self.padding[:2], self.dilation[:2],
                                            self.groups)


class _unpoolLayer(nn.ConvTranspose3d):
    """Unpooling as a 1 -> 1 channel transposed synapse with constant weights ``1.1 * theta`` on the
    tensor viewed as (N, 1, C*H, W, T) (src/slayer.py:645-748)."""

    def __init__(self, theta, kernelSize, stride=None, padding=0, dilation=1, preHookFx=None):
        kernel = _hw(kernelSize, "kernelSize")
        super().__init__(1, 1, kernel, _hw(stride, "stride", kernel), _hw(padding, "padding"), 0, 1, False,
                         _hw(dilation, "dilation"))
        self.weight = _poolWeight(theta, self.weight.shape)
        self.preHookFx = preHookFx

    def forward(self, input):
        N, C, H, W, T = input.shape
        weight = self.weight if self.preHookFx is None else self.preHookFx(self.weight)
        result = synapse.synapseConvTranspose(input.reshape(N, 1, C * H, W, T), weight, self.stride[:2],
                                              self.padding[:2], self.dilation[:2], 1)
        return result.reshape(result.shape[0], C, -1, result.shape[3], result.shape[4])


class _dropoutLayer(nn.Dropout3d):
    """Dropout over whole neurons: the tensor is viewed as (N, C*H*W, 1, 1, T) so that ``dropout3d``
    zeroes entire time rows (src/slayer.py:748-759)."""

    def forward(self, input):
        shape = input.shape
        return F.dropout3d(input.reshape(shape[0], -1, 1, 1, shape[-1]), self.p, self.training,
                           self.inplace).reshape(shape)


class _spikeFunction(torch.autograd.Function):
    """Forward: ``slayerCuda.getSpikes``; backward: spike-function surrogate gradient
    ``gradOutput * scaleRho/(tauRho*theta) * exp(-|u - theta| / (tauRho*theta))``
    (src/slayer.py:817-865)."""

    @staticmethod
    def forward(ctx, membranePotential, refractoryResponse, neuron, Ts):
        theta = neuron["theta"]
        # A contiguous input IS the buffer the kernel updates in place; a non-contiguous one is
        # copied and keeps its values.  Either way the tensor saved for backward is the
        # caller's, exactly as in the reference.
        spikes = slayerCuda.getSpikes(membranePotential.contiguous(), refractoryResponse, theta, Ts)
        ctx.save_for_backward(membranePotential)
        ctx.set_materialize_grads(False)   # no gradient for the spikes: no kernel, not a tensor of zeros through it
        ctx.theta = float(theta)
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        return spikes

    @staticmethod
    def backward(ctx, gradOutput):
        if gradOutput is None:
            return None, None, None, None
        (membranePotential,) = ctx.saved_tensors
        gradInput = slayerCuda.spikeBackward(gradOutput.contiguous(), membranePotential.contiguous(),
                                             ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale)
        return gradInput, None, None, None


class _spikeDelayedFunction(torch.autograd.Function):
    """``_spikeFunction`` followed by ``_delayFunction`` / ``_delayFunctionNoGradient``
    (src/slayer.py:817-865, 930-979) as one Function over ``slayerCuda.getSpikesDelayed`` and
    ``slayerCuda.spikeBackwardDelayed``.  ``delay`` is a number or a tensor; a tensor that requires
    grad gets the delay gradient of ``_delayFunction.backward``."""

    @staticmethod
    def forward(ctx, membranePotential, refractoryResponse, neuron, Ts, delay, delayTs):
        theta = neuron["theta"]
        table = delay.detach().to(device=membranePotential.device, dtype=membranePotential.dtype).contiguous() \
            if isinstance(delay, torch.Tensor) else delay
        spikes = slayerCuda.getSpikesDelayed(membranePotential.contiguous(), refractoryResponse, theta, Ts, table,
                                             delayTs)
        ctx.learn = isinstance(delay, torch.Tensor) and delay.requires_grad
        ctx.save_for_backward(membranePotential, *((spikes,) if ctx.learn else ()))
        ctx.delay = table
        ctx.delayShape = tuple(delay.shape) if isinstance(delay, torch.Tensor) else None
        ctx.delayTs = float(delayTs)
        ctx.theta = float(theta)
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        return spikes

    @staticmethod
    def backward(ctx, gradOutput):
        membranePotential = ctx.saved_tensors[0]
        gradOutput = gradOutput.contiguous()
        gradDelay = None
        if ctx.learn:
            gradDelay = slayerCuda.delayGrad(ctx.saved_tensors[1], gradOutput, ctx.delayTs).reshape(ctx.delayShape)
        gradInput = slayerCuda.spikeBackwardDelayed(gradOutput, membranePotential.contiguous(), ctx.theta,
                                                    ctx.pdfTimeConstant, ctx.pdfScale, ctx.delay, ctx.delayTs)
        return gradInput, None, None, None, gradDelay, None


def _fresh_spikes(spike):
    """(membranePotential, theta, pdfTimeConstant, pdfScale) when ``spike`` is what ``spikeLayer.spike`` has just
    returned for that potential - its own output, untouched, with the graph being recorded - else None."""
    origin = _spikeNotes.get(spike) if PAIR_SPIKE_PSP else None
    if origin is None or not torch.is_grad_enabled() or not spike.requires_grad or spike._version != origin[4] \
            or not isinstance(spike.grad_fn, _spikeFunction._backward_cls) or not _unobserved(spike):
        return None
    membranePotential = origin[0]()
    # (a potential changed in place after spike() must reach the spike function's own backward pass, whose saved
    # tensor then raises; the paired kernel would silently use the changed values)
    if membranePotential is None or membranePotential.shape != spike.shape or not membranePotential.is_contiguous() \
            or membranePotential._version != origin[5]:
        return None
    return membranePotential, origin[1], origin[2], origin[3]


# The pairing notes live beside the tensors, not on them: a tensor with Python attributes is pickled with them
# (torch.save of a layer's output would carry the note, or fail on it), and an entry goes when its tensor does.
_pspNotes = WeakTensorKeyDictionary()     # psp() output -> (its input, kernel, (tau, mult), version)
_spikeNotes = WeakTensorKeyDictionary()   # spike() output -> (weak potential, theta, pdf tau, pdf scale, versions)


def _unobserved(tensor):
    """False when the caller watches this tensor's gradient (``retain_grad`` or a hook registered on it): the paired
    kernels route the gradient around the tensor, so such a tensor keeps the separate Functions."""
    return not tensor.retains_grad and not tensor._backward_hooks


def _recursion_serves(x):
    """Shapes that ``slayerCuda.pspAlpha`` runs as a recursion (others it hands to conv / corr itself): rows of at most
    512 samples in a tensor of whole 16-byte vectors, and longer rows of whole vectors (taken in pieces)."""
    T = x.shape[-1]
    return x.numel() % 4 == 0 if T <= 512 else T % 4 == 0


class _pspSpikeFunction(torch.autograd.Function):
    """``_pspFunction`` followed by ``_spikeFunction`` (src/slayer.py:817-899) as one Function:
    forward is ``slayerCuda.pspSpike``; backward is the spike function's surrogate gradient
    followed by the correlation with the SRM kernel, also in one kernel."""

    @staticmethod
    def forward(ctx, input, srmKernel, refractoryResponse, neuron, Ts, alpha=None):
        if alpha is None or not _recursion_serves(input):
            spikes, membranePotential = slayerCuda.pspSpike(input.contiguous(), srmKernel, refractoryResponse,
                                                            neuron["theta"], Ts)
        else:
            # the alpha kernel as a recursion over time, then the spike kernel: two memory streams, which together
            # take less time than the one kernel that sums over the taps (and the very values of psp() + spike())
            membranePotential = slayerCuda.pspAlpha(input.contiguous(), srmKernel, alpha[0], alpha[1], Ts, causal=True)
            spikes = slayerCuda.getSpikes(membranePotential, refractoryResponse, neuron["theta"], Ts)
        ctx.save_for_backward(membranePotential, srmKernel)
        ctx.alpha = alpha if alpha is not None and _recursion_serves(input) else None
        ctx.theta = float(neuron["theta"])
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        ctx.Ts = float(Ts)
        return spikes

    @staticmethod
    def backward(ctx, gradOutput):
        membranePotential, srmKernel = ctx.saved_tensors
        if ctx.alpha is None:
            gradInput = slayerCuda.spikeBackwardCorr(gradOutput.contiguous(), membranePotential, srmKernel, ctx.theta,
                                                     ctx.pdfTimeConstant, ctx.pdfScale, ctx.Ts)
        else:
            gradInput = slayerCuda.spikeBackwardPspAlpha(gradOutput.contiguous(), membranePotential, srmKernel,
                                                         ctx.alpha[0], ctx.alpha[1], ctx.theta, ctx.pdfTimeConstant,
                                                         ctx.pdfScale, ctx.Ts)
        return gradInput, None, None, None, None, None


class _pspFunction(torch.autograd.Function):
    """Forward: causal conv with the SRM kernel; backward: correlation with the same kernel;
    the kernel itself gets no gradient (src/slayer.py:875-899).  ``alpha`` = (tau, mult) when the
    kernel is known to be that alpha kernel: both then run as recursions over time."""

    @staticmethod
    def forward(ctx, spike, filter, Ts, alpha=None):
        if alpha is not None and not _recursion_serves(spike):
            alpha = None
        if alpha is None:
            psp = slayerCuda.conv(spike.contiguous(), filter, Ts)
        else:
            psp = slayerCuda.pspAlpha(spike.contiguous(), filter, alpha[0], alpha[1], Ts, causal=True)
        ctx.save_for_backward(filter)
        ctx.set_materialize_grads(False)   # no gradient for the signal: no kernel, not a tensor of zeros through it
        ctx.Ts = float(Ts)
        ctx.alpha = alpha
        return psp

    @staticmethod
    def backward(ctx, gradOutput):
        if gradOutput is None:
            return None, None, None, None
        (filter,) = ctx.saved_tensors
        if ctx.alpha is None:
            gradInput = slayerCuda.corr(gradOutput.contiguous(), filter, ctx.Ts)
        else:
            gradInput = slayerCuda.pspAlpha(gradOutput.contiguous(), filter, ctx.alpha[0], ctx.alpha[1], ctx.Ts,
                                            causal=False)
        return gradInput, None, None, None


class _spikeOfPspFunction(torch.autograd.Function):
    """``_spikeFunction`` (src/slayer.py:817-865) for a membrane potential that ``_pspFunction`` has just produced
    from ``pspInput`` with the alpha kernel as a recursion.  Forward: the spike function.  Backward: the gradient
    goes to ``pspInput`` directly - surrogate gradient, then the correlation of ``_pspFunction.backward``
    (src/slayer.py:888-893), in one kernel - and nothing to ``membranePotential``, whose producer then only
    carries what reaches the potential from elsewhere."""

    @staticmethod
    def forward(ctx, membranePotential, pspInput, refractoryResponse, filter, neuron, Ts, alpha):
        spikes = slayerCuda.getSpikes(membranePotential, refractoryResponse, neuron["theta"], Ts)
        ctx.save_for_backward(membranePotential, filter)
        ctx.set_materialize_grads(False)
        ctx.alpha, ctx.Ts = alpha, float(Ts)
        ctx.theta = float(neuron["theta"])
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        return spikes

    @staticmethod
    def backward(ctx, gradOutput):
        grad = None
        if gradOutput is not None and ctx.needs_input_grad[1]:
            membranePotential, filter = ctx.saved_tensors
            grad = slayerCuda.spikeBackwardPspAlpha(gradOutput.contiguous(), membranePotential, filter, ctx.alpha[0],
                                                    ctx.alpha[1], ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale, ctx.Ts)
        return None, grad, None, None, None, None, None


class _pspOfSpikeFunction(torch.autograd.Function):
    """``_pspFunction`` (src/slayer.py:875-899) for a spike tensor that ``_spikeFunction`` has just produced from
    ``membranePotential``, with the alpha kernel as a recursion.  Forward: the PSP filter.  Backward: the
    gradient goes to ``membranePotential`` directly - correlation, then the spike function's surrogate
    gradient (src/slayer.py:858-865), in one kernel - and nothing to ``spike``, whose own backward pass then
    only carries what reaches the spikes from elsewhere."""

    @staticmethod
    def forward(ctx, spike, membranePotential, filter, Ts, alpha, theta, pdfTimeConstant, pdfScale):
        psp = slayerCuda.pspAlpha(spike.contiguous(), filter, alpha[0], alpha[1], Ts, causal=True)
        ctx.save_for_backward(membranePotential, filter)
        ctx.Ts, ctx.alpha = float(Ts), alpha
        ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale = theta, pdfTimeConstant, pdfScale
        return psp

    @staticmethod
    def backward(ctx, gradOutput):
        membranePotential, filter = ctx.saved_tensors
        grad = None
        if ctx.needs_input_grad[1]:
            grad = slayerCuda.pspSpikeBackwardAlpha(gradOutput.contiguous(), None, membranePotential, filter, ctx.alpha[0],
                                                    ctx.alpha[1], ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale, ctx.Ts)
        return None, grad, None, None, None, None, None, None


class _spikePspFunction(torch.autograd.Function):
    """``_spikeFunction`` followed by ``_pspFunction`` (src/slayer.py:817-899) with both results as outputs.
    Forward: ``slayerCuda.getSpikes``, then the PSP filter; backward: correlation of the PSP gradient, plus the
    gradient that reaches the spikes directly, times the surrogate gradient - one kernel when the PSP kernel
    is the layer's alpha kernel and the recursion serves the shape, else the three calls."""

    @staticmethod
    def forward(ctx, membranePotential, refractoryResponse, filter, neuron, Ts, alpha=None):
        theta = neuron["theta"]
        ctx.set_materialize_grads(False)   # an output that was not used brings None, not a tensor of zeros
        spikes = slayerCuda.getSpikes(membranePotential.contiguous(), refractoryResponse, theta, Ts)
        if alpha is not None and not _recursion_serves(spikes):
            alpha = None
        if alpha is None:
            psp = slayerCuda.conv(spikes, filter, Ts)
        else:
            psp = slayerCuda.pspAlpha(spikes, filter, alpha[0], alpha[1], Ts, causal=True)
        ctx.save_for_backward(membranePotential, filter)
        ctx.theta = float(theta)
        ctx.pdfTimeConstant = float(neuron["tauRho"] * neuron["theta"])
        ctx.pdfScale = float(neuron["scaleRho"])
        ctx.Ts = float(Ts)
        ctx.alpha = alpha
        return spikes, psp

    @staticmethod
    def backward(ctx, gradSpikes, gradPsp):
        membranePotential, filter = ctx.saved_tensors
        u = membranePotential.contiguous()
        if gradPsp is None and gradSpikes is None:
            return None, None, None, None, None, None
        if gradPsp is None:      # only the spikes were used
            grad = slayerCuda.spikeBackward(gradSpikes.contiguous(), u, ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale)
        elif ctx.alpha is not None:
            grad = slayerCuda.pspSpikeBackwardAlpha(gradPsp.contiguous(), None if gradSpikes is None else gradSpikes.contiguous(),
                                                    u, filter, ctx.alpha[0], ctx.alpha[1], ctx.theta, ctx.pdfTimeConstant,
                                                    ctx.pdfScale, ctx.Ts)
        else:
            grad = slayerCuda.corr(gradPsp.contiguous(), filter, ctx.Ts)
            if gradSpikes is not None:
                grad = grad + gradSpikes
            grad = slayerCuda.spikeBackward(grad, u, ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale)
        return grad, None, None, None, None, None


class _delayLayer(nn.Module):
    """Learnable delay, one per neuron (C,H,W) or one per channel when the input's H and W
    exceed the parameter's (src/slayer.py:901-928).  Initialised U[0,1)."""

    def __init__(self, inputSize, Ts):
        super().__init__()
        if isinstance(inputSize, int):
            shape = (inputSize, 1, 1)
        elif len(inputSize) == 3:
            shape = (inputSize[0], inputSize[1], inputSize[2])
        else:
            raise Exception("inputSize can only be 1 or 2 dimension. It was: {}".format(inputSize))
        self.delay = nn.Parameter(torch.rand(shape), requires_grad=True)
        self.Ts = Ts

    def forward(self, input):
        N, C, H, W, Ns = input.shape
        table = self.delay.repeat((1, H, W)) if input.numel() != self.delay.numel() * Ns * N else self.delay
        origin = _fresh_spikes(input)
        if origin is not None:
            return _delayOfSpikeFunction.apply(input, origin[0], table, self.Ts, True, *origin[1:])
        return _delayFunction.apply(input, table, self.Ts)


class _delayFunction(torch.autograd.Function):
    """Shift by a per-neuron delay table with gradients for both the input (shift by the
    negated delay) and the delays (src/slayer.py:930-957)."""

    @staticmethod
    def forward(ctx, input, delay, Ts):
        output = slayerCuda.shift(input.contiguous(), delay.data.contiguous(), Ts)
        ctx.save_for_backward(output, delay.data)
        ctx.Ts = float(Ts)
        return output

    @staticmethod
    def backward(ctx, gradOutput):
        output, delay = ctx.saved_tensors
        gradOutput = gradOutput.contiguous()
        gradDelay = slayerCuda.delayGrad(output, gradOutput, ctx.Ts).reshape(gradOutput.shape[1:-1])
        gradInput = slayerCuda.shift(gradOutput, delay.contiguous(), ctx.Ts, sign=-1.0)
        return gradInput, gradDelay, None


class _delayOfSpikeFunction(torch.autograd.Function):
    """``_delayFunction`` / ``_delayFunctionNoGradient`` (src/slayer.py:930-979) for a spike tensor that
    ``_spikeFunction`` has just produced from ``membranePotential``.  Forward: the shift.  Backward: the gradient
    goes to ``membranePotential`` directly - shifted back and multiplied by the spike function's surrogate gradient
    (src/slayer.py:858-865) in one kernel - and nothing to ``spike``; a learnable delay table (``learn``) gets the
    delay gradient as in ``_delayFunction``."""

    @staticmethod
    def forward(ctx, spike, membranePotential, delay, Ts, learn, theta, pdfTimeConstant, pdfScale):
        table = delay.detach().to(device=spike.device, dtype=spike.dtype).contiguous() \
            if isinstance(delay, torch.Tensor) else delay
        output = slayerCuda.shift(spike.contiguous(), table, Ts)
        ctx.learn = bool(learn)
        ctx.save_for_backward(membranePotential, *((output,) if ctx.learn else ()))
        ctx.delay, ctx.Ts = table, float(Ts)
        ctx.delayShape = tuple(delay.shape) if isinstance(delay, torch.Tensor) else None
        ctx.theta, ctx.pdfTimeConstant, ctx.pdfScale = theta, pdfTimeConstant, pdfScale
        return output

    @staticmethod
    def backward(ctx, gradOutput):
        membranePotential = ctx.saved_tensors[0]
        gradOutput = gradOutput.contiguous()
        gradDelay = grad = None
        if ctx.learn and ctx.needs_input_grad[2]:
            gradDelay = slayerCuda.delayGrad(ctx.saved_tensors[1], gradOutput, ctx.Ts).reshape(ctx.delayShape)
        if ctx.needs_input_grad[1]:
            grad = slayerCuda.spikeBackwardDelayed(gradOutput, membranePotential, ctx.theta, ctx.pdfTimeConstant,
                                                   ctx.pdfScale, ctx.delay, ctx.Ts)
        return None, grad, gradDelay, None, None, None, None, None


class _delayFunctionNoGradient(torch.autograd.Function):
    """Shift by a fixed delay (number or tensor); backward shifts the gradient by the negated
    delay (src/slayer.py:959-979)."""

    @staticmethod
    def forward(ctx, input, delay, Ts=1):
        if isinstance(delay, torch.Tensor):
            delay = delay.detach().to(device=input.device, dtype=input.dtype).contiguous()
        output = slayerCuda.shift(input.contiguous(), delay, Ts)
        ctx.delay = delay
        ctx.Ts = float(Ts)
        return output

    @staticmethod
    def backward(ctx, gradOutput):
        return slayerCuda.shift(gradOutput.contiguous(), ctx.delay, ctx.Ts, sign=-1.0), None, None

"""``slayerLoihiCuda`` for MI355X: the one callable of the reference's pybind11 extension
(src/cuda/slayerLoihiKernels.cu:48-51), implemented over the C ABI of ``libslayer_hip.so``.

``getSpikesDelayed`` has no counterpart in the reference extension: it is ``getSpikes`` with the
``delayShift`` that follows it in Loihi networks (src/auto/loihi.py:67-69) fused in and with
optional voltage / current outputs.
"""
import operator

import torch

from . import _lib
from .slayerCuda import _check_input, _on_device_of, _ptr, _rows

__all__ = ["getSpikes", "getSpikesDelayed", "quantize", "MAX_FUSED_DELAY"]

MAX_FUSED_DELAY = 31   # longest spike delay (samples) that getSpikesDelayed fuses into the neuron kernel


def _unsigned(x, name):
    """pybind11's ``unsigned`` conversion: integers (anything with ``__index__``) >= 0 only."""
    if isinstance(x, torch.Tensor):
        if x.numel() != 1 or x.is_floating_point():
            raise TypeError("%s must be a non-negative integer" % name)
        x = int(x)
    try:
        v = operator.index(x)
    except TypeError:
        raise TypeError("%s must be a non-negative integer, got %s" % (name, type(x).__name__))
    if v < 0 or v > 0xFFFFFFFF:
        raise TypeError("%s must fit an unsigned 32 bit integer, got %d" % (name, v))
    return v


def _neuron_args(wgtExp, theta, iDecay, vDecay, refDelay):
    wgtExp = _unsigned(wgtExp, "wgtExp")
    theta = _unsigned(theta, "theta")
    iDecay = _unsigned(iDecay, "iDecay")
    vDecay = _unsigned(vDecay, "vDecay")
    refDelay = _unsigned(refDelay, "refDelay")
    if refDelay == 0:
        # the reference kernel reads a spike sample it has not written yet in this case
        raise ValueError("refDelay must be at least 1")
    if wgtExp > 25:
        raise ValueError("wgtExp must be at most 25 (weight scale 1 << (6 + wgtExp) is 32 bit)")
    if theta > 0x7FFFFFFF:
        raise ValueError("theta must fit a signed 32 bit integer")
    return wgtExp, theta, iDecay, vDecay, refDelay


def getSpikes(weightedSpikes, wgtExp, theta, iDecay, vDecay, refDelay):
    """Loihi CUBA neuron on ``weightedSpikes`` (any shape, time last).  Returns
    ``[spike, voltage, current]`` (src/cuda/slayerLoihiKernels.cu:12-46)."""
    _check_input(weightedSpikes, "weightedSpikes")
    wgtExp, theta, iDecay, vDecay, refDelay = _neuron_args(wgtExp, theta, iDecay, vDecay, refDelay)
    lib = _lib.load()
    spike = torch.empty_like(weightedSpikes)
    voltage = torch.empty_like(weightedSpikes)
    current = torch.empty_like(weightedSpikes)
    n, T = _rows(weightedSpikes)
    with _on_device_of(weightedSpikes) as stream:
        _lib.check(lib.slayer_loihi_get_spikes_f32(_ptr(spike), _ptr(voltage), _ptr(current),
                                                   _ptr(weightedSpikes), n, T, wgtExp, theta, iDecay,
                                                   vDecay, refDelay, stream),
                   "slayer_loihi_get_spikes_f32")
    return [spike, voltage, current]


def getSpikesDelayed(weightedSpikes, wgtExp, theta, iDecay, vDecay, refDelay, delaySteps=0, voltage=True,
                     current=True):
    """:func:`getSpikes` whose spike output comes ``delaySteps`` samples late (zeros before), i.e.
    followed by ``shift(spike, delaySteps)``, in one kernel; ``0 <= delaySteps <= MAX_FUSED_DELAY``.
    Voltage and current are not shifted; with ``voltage=False`` / ``current=False`` they are not
    computed into memory at all and ``None`` is returned in their place."""
    _check_input(weightedSpikes, "weightedSpikes")
    wgtExp, theta, iDecay, vDecay, refDelay = _neuron_args(wgtExp, theta, iDecay, vDecay, refDelay)
    delaySteps = _unsigned(delaySteps, "delaySteps")
    if delaySteps > MAX_FUSED_DELAY:
        raise ValueError("delaySteps must be at most %d; shift separately for longer delays" % MAX_FUSED_DELAY)
    lib = _lib.load()
    spike = torch.empty_like(weightedSpikes)
    volt = torch.empty_like(weightedSpikes) if voltage else None
    curr = torch.empty_like(weightedSpikes) if current else None
    n, T = _rows(weightedSpikes)
    with _on_device_of(weightedSpikes) as stream:
        _lib.check(lib.slayer_loihi_get_spikes_delayed_f32(
            _ptr(spike), _ptr(volt) if voltage else None, _ptr(curr) if current else None,
            _ptr(weightedSpikes), n, T, wgtExp, theta, iDecay, vDecay, refDelay, delaySteps, stream),
            "slayer_loihi_get_spikes_delayed_f32")
    return [spike, volt, curr]


def quantize(weights, step):
    """``torch.round(weights / step) * step`` (src/quantizeParams.py:17-23) from one kernel, the same values
    bit for bit.  Has no counterpart in the reference extension."""
    _check_input(weights, "weights")
    step = float(step)
    if step == 0.0 or step != step:
        raise ValueError("step must be a non-zero number")
    lib = _lib.load()
    out = torch.empty_like(weights)
    with _on_device_of(weights) as stream:
        _lib.check(lib.slayer_quantize_f32(_ptr(out), _ptr(weights), weights.numel(), step, stream), "slayer_quantize_f32")
    return out

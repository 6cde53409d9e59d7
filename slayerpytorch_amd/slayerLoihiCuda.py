"""``slayerLoihiCuda`` for MI355X: the one callable of the reference's pybind11 extension
(src/cuda/slayerLoihiKernels.cu:48-51), implemented over the C ABI of ``libslayer_hip.so``.
"""
import operator

import torch

from . import _lib
from .slayerCuda import _check_input, _on_device_of, _ptr, _rows

__all__ = ["getSpikes"]


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


def getSpikes(weightedSpikes, wgtExp, theta, iDecay, vDecay, refDelay):
    """Loihi CUBA neuron on ``weightedSpikes`` (any shape, time last).  Returns
    ``[spike, voltage, current]`` (src/cuda/slayerLoihiKernels.cu:12-46)."""
    _check_input(weightedSpikes, "weightedSpikes")
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

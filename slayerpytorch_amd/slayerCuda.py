"""``slayerCuda`` for MI355X: same callables as the reference's pybind11 extension
(src/cuda/slayerKernels.cu:136-145), implemented over the C ABI of ``libslayer_hip.so``.

===================================  ==========================================================
callable                             reference binding it replaces
===================================  ==========================================================
``getSpikes(u, nu, theta, Ts)``      ``getSpikesCuda``  src/cuda/slayerKernels.cu:14-39
``conv(input, filter, Ts)``          ``convCuda``       src/cuda/slayerKernels.cu:41-57
``corr(input, filter, Ts)``          ``corrCuda``       src/cuda/slayerKernels.cu:59-75
``shift(input, lut[, Ts])``          ``shiftCuda`` / ``shift1Cuda``     :77-112
``shift(input, delay[, Ts])``        ``shiftFlCuda`` / ``shiftFl1Cuda`` :114-134
===================================  ==========================================================

Argument checks mirror the reference's ``CHECK_INPUT`` / ``CHECK_DEVICE`` assertions and are
made before anything is launched, so they can be exercised without a GPU.  Scalars may be
Python numbers or 0-dim tensors, as with pybind11's float conversion.  Outputs are allocated
with ``torch.empty_like``; kernels are enqueued on PyTorch's current stream of the tensor's
device and never synchronise with the host.

``spikeBackward``, ``spikeBackwardCorr``, ``pspSpike``, ``getSpikesDelayed``, ``spikeBackwardDelayed``,
``delayGrad`` and the ``sign`` argument
of ``shift`` have no counterpart in the reference extension: they are the fused forms of the
elementwise chains in ``_spikeFunction.backward`` / ``_delayFunction.backward``
(src/slayer.py:857-865, 944-957), of ``slayerLoihi._spike.backward`` (src/slayerLoihi.py:278-283)
and of the call pairs ``spike(psp(x))`` and ``delayShift(spike(u), d)``.
"""
import numbers

import torch

from . import _lib

__all__ = ["getSpikes", "conv", "corr", "shift", "spikeBackward", "spikeBackwardCorr", "pspSpike", "delayGrad",
           "getSpikesDelayed", "spikeBackwardDelayed", "spikeLoss", "pspAlpha", "spikeBackwardPspAlpha",
           "pspSpikeBackwardAlpha"]


def _check_input(x, name):
    if not isinstance(x, torch.Tensor):
        raise TypeError("%s must be a torch.Tensor, got %s" % (name, type(x).__name__))
    if not x.is_cuda:
        raise RuntimeError("%s must be a CUDA tensor" % name)
    if not x.is_contiguous():
        raise RuntimeError("%s must be contiguous" % name)
    if x.dtype != torch.float32:
        raise RuntimeError("expected scalar type Float but found %s for %s" % (x.dtype, name))


def _check_device(x, y, xname, yname):
    if x.device.index != y.device.index:
        raise RuntimeError("%s and %s must be in same CUDA device" % (xname, yname))


def _scalar(x, name):
    if isinstance(x, torch.Tensor):
        if x.numel() != 1:
            raise TypeError("%s must be a number or a one-element tensor" % name)
        return float(x)
    if isinstance(x, numbers.Real):
        return float(x)
    if isinstance(x, (str, bytes)):
        raise TypeError("%s must be a number, got %s" % (name, type(x).__name__))
    try:
        return float(x)   # numpy scalars and other objects with __float__
    except Exception:
        raise TypeError("%s must be a number, got %s" % (name, type(x).__name__))


def _ptr(x):
    return x.data_ptr() if x.numel() else None


def _rows(x):
    T = x.shape[-1] if x.dim() else 1
    return (x.numel() // T if T else 0), T


def _raw_stream(index):
    """Raw handle of PyTorch's current stream on device ``index``."""
    get = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # skips building a Stream object
    return get(index) if get is not None else torch.cuda.current_stream(index).cuda_stream


class _on_device_of:
    """Makes the tensor's device current (like the reference's cudaSetDevice) and yields the
    raw handle of PyTorch's current stream there."""
    __slots__ = ("index", "guard")

    def __init__(self, x):
        self.index = x.device.index
        self.guard = None

    def __enter__(self):
        if self.index != torch.cuda.current_device():
            self.guard = torch.cuda.device(self.index)
            self.guard.__enter__()
        return _raw_stream(self.index)

    def __exit__(self, *exc):
        if self.guard is not None:
            return self.guard.__exit__(*exc)
        return False


def getSpikes(d_u, d_nu, theta, Ts):
    """Spikes of the membrane potential ``d_u`` (N,C,H,W,T); ``d_u`` is updated IN PLACE with
    the refractory response ``d_nu`` of every spike.  Returns the spike tensor (``1/Ts`` at
    spikes)."""
    _check_input(d_u, "d_u")
    _check_input(d_nu, "d_nu")
    _check_device(d_u, d_nu, "d_u", "d_nu")
    if d_u.dim() < 4:
        raise IndexError("Dimension out of range (getSpikes expects a 5 dimensional N,C,H,W,T tensor, "
                         "got %d dimensions)" % d_u.dim())
    if d_u.dim() != 5:
        raise RuntimeError("getSpikes expects a 5 dimensional (N,C,H,W,T) tensor, got %d dimensions"
                           % d_u.dim())
    theta = _scalar(theta, "theta")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    d_s = torch.empty_like(d_u)
    n, T = _rows(d_u)
    nuSize = d_nu.shape[-1] if d_nu.dim() else 1
    with _on_device_of(d_u) as stream:
        _lib.check(lib.slayer_get_spikes_f32(_ptr(d_s), _ptr(d_u), _ptr(d_nu), n, T, nuSize, theta, Ts,
                                             stream), "slayer_get_spikes_f32")
    return d_s


def _fir(entry, name, input, filter, Ts):
    _check_input(input, "input")
    _check_input(filter, "filter")
    _check_device(input, filter, "input", "filter")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    output = torch.empty_like(input)
    n, T = _rows(input)
    with _on_device_of(input) as stream:
        _lib.check(getattr(lib, entry)(_ptr(output), _ptr(input), _ptr(filter), n, T, filter.numel(), Ts,
                                       stream), entry)
    return output


def conv(input, filter, Ts):
    """Causal convolution in time (last axis) of every neuron row with ``filter``, times ``Ts``."""
    return _fir("slayer_conv_f32", "conv", input, filter, Ts)


def corr(input, filter, Ts):
    """Anti-causal correlation in time (adjoint of :func:`conv`), times ``Ts``."""
    return _fir("slayer_corr_f32", "corr", input, filter, Ts)


def pspAlpha(input, filter, tau, mult, Ts, causal=True):
    """``conv(input, filter, Ts)`` (``causal``) or ``corr(input, filter, Ts)`` for a ``filter`` that holds the
    alpha kernel ``mult * t/tau * exp(1 - t/tau)`` sampled at ``t = 0, Ts, 2 Ts, ...`` (what
    ``spikeLayer.calculateSrmKernel`` builds), computed as a recursion over time instead of a sum over
    the taps.  Agrees with ``conv`` / ``corr`` to rounding; see ``slayer_psp_alpha_f32`` in the header
    for the bound.  The caller vouches for ``filter`` being that kernel."""
    _check_input(input, "input")
    _check_input(filter, "filter")
    _check_device(input, filter, "input", "filter")
    tau, mult, Ts = _scalar(tau, "tau"), _scalar(mult, "mult"), _scalar(Ts, "Ts")
    if filter.numel() < 1:
        raise RuntimeError("pspAlpha needs a filter of at least one tap")
    lib = _lib.load()
    output = torch.empty_like(input)
    n, T = _rows(input)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_psp_alpha_f32(_ptr(output), _ptr(input), _ptr(filter), n, T, filter.numel(), tau, mult,
                                            Ts, 1 if causal else 0, stream), "slayer_psp_alpha_f32")
    return output


def spikeBackwardPspAlpha(gradOutput, membranePotential, filter, tauSr, mult, theta, tau, scale, Ts):
    """:func:`spikeBackwardCorr` for a ``filter`` that holds the alpha kernel of :func:`pspAlpha`
    (``tauSr``, ``mult``): the surrogate gradient (``theta``, ``tau``, ``scale`` as in
    :func:`spikeBackward`) and the correlation as a recursion over time, in one kernel."""
    _check_input(gradOutput, "gradOutput")
    _check_input(membranePotential, "membranePotential")
    _check_input(filter, "filter")
    _check_device(gradOutput, membranePotential, "gradOutput", "membranePotential")
    _check_device(gradOutput, filter, "gradOutput", "filter")
    if gradOutput.shape != membranePotential.shape:
        raise RuntimeError("gradOutput and membranePotential must have the same shape")
    if filter.numel() < 1:
        raise RuntimeError("spikeBackwardPspAlpha needs a filter of at least one tap")
    tauSr, mult, theta, tau = _scalar(tauSr, "tauSr"), _scalar(mult, "mult"), _scalar(theta, "theta"), _scalar(tau, "tau")
    scale, Ts = _scalar(scale, "scale"), _scalar(Ts, "Ts")
    lib = _lib.load()
    gradInput = torch.empty_like(gradOutput)
    n, T = _rows(gradOutput)
    with _on_device_of(gradOutput) as stream:
        _lib.check(lib.slayer_spike_bwd_psp_alpha_f32(_ptr(gradInput), _ptr(gradOutput), _ptr(membranePotential), _ptr(filter),
                                                      n, T, filter.numel(), tauSr, mult, theta, tau, scale, Ts, stream),
                   "slayer_spike_bwd_psp_alpha_f32")
    return gradInput


def pspSpikeBackwardAlpha(gradPsp, gradSpike, membranePotential, filter, tauSr, mult, theta, tau, scale, Ts):
    """Backward pass of ``psp(spike(u))`` for a ``filter`` that holds the alpha kernel of :func:`pspAlpha`
    (``tauSr``, ``mult``): ``spikeBackward(corr(gradPsp, filter, Ts) + gradSpike, u, theta, tau, scale)`` in one
    kernel; ``gradSpike`` (the gradient that reaches the spikes directly) may be ``None``.  Shapes the
    recursion does not serve take those three calls."""
    _check_input(gradPsp, "gradPsp")
    _check_input(membranePotential, "membranePotential")
    _check_input(filter, "filter")
    _check_device(gradPsp, membranePotential, "gradPsp", "membranePotential")
    _check_device(gradPsp, filter, "gradPsp", "filter")
    if gradPsp.shape != membranePotential.shape:
        raise RuntimeError("gradPsp and membranePotential must have the same shape")
    if gradSpike is not None:
        _check_input(gradSpike, "gradSpike")
        _check_device(gradPsp, gradSpike, "gradPsp", "gradSpike")
        if gradSpike.shape != gradPsp.shape:
            raise RuntimeError("gradSpike and gradPsp must have the same shape")
    if filter.numel() < 1:
        raise RuntimeError("pspSpikeBackwardAlpha needs a filter of at least one tap")
    tauSr, mult, theta, tau = _scalar(tauSr, "tauSr"), _scalar(mult, "mult"), _scalar(theta, "theta"), _scalar(tau, "tau")
    scale, Ts = _scalar(scale, "scale"), _scalar(Ts, "Ts")
    lib = _lib.load()
    gradInput = torch.empty_like(gradPsp)
    n, T = _rows(gradPsp)
    with _on_device_of(gradPsp) as stream:
        status = lib.slayer_psp_spike_bwd_alpha_f32(_ptr(gradInput), _ptr(gradPsp),
                                                    _ptr(gradSpike) if gradSpike is not None else None,
                                                    _ptr(membranePotential), _ptr(filter), n, T, filter.numel(), tauSr, mult,
                                                    theta, tau, scale, Ts, stream)
    if status == 2:  # not a shape for the recursion
        grad = corr(gradPsp, filter, Ts)
        if gradSpike is not None:
            grad = grad + gradSpike
        return spikeBackward(grad, membranePotential, theta, tau, scale)
    _lib.check(status, "slayer_psp_spike_bwd_alpha_f32")
    return gradInput


def shift(input, shiftLUT, Ts=1.0, sign=1.0):
    """Shifts every neuron row in time by ``int(delay / Ts)`` samples (zero fill).

    ``shiftLUT`` is a number (one delay for all rows), a one-element tensor (same, read on the
    device) or a tensor with one delay per neuron of a batch item (``numel == C*H*W``).
    ``sign`` (+1/-1, extension) multiplies the delays, for the backward shift.
    """
    _check_input(input, "input")
    sign = float(sign)
    if isinstance(shiftLUT, torch.Tensor):
        _check_input(shiftLUT, "shiftLUT")
        _check_device(input, shiftLUT, "input", "shiftLUT")
        Ts = _scalar(Ts, "Ts")
        n, T = _rows(input)
        if shiftLUT.numel() == 1:
            nBatch, nPerBatch = 1, n
        else:
            nBatch = input.shape[0]
            nPerBatch = (n // nBatch) if nBatch else 0
            if shiftLUT.numel() != nPerBatch:
                raise RuntimeError("shift and number of neurons must be same")
        lib = _lib.load()
        output = torch.empty_like(input)
        with _on_device_of(input) as stream:
            _lib.check(lib.slayer_shift_lut_f32(_ptr(output), _ptr(input), _ptr(shiftLUT),
                                                shiftLUT.numel(), nBatch, nPerBatch, T, Ts, sign, stream),
                       "slayer_shift_lut_f32")
        return output
    delay = _scalar(shiftLUT, "shiftLUT")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    output = torch.empty_like(input)
    n, T = _rows(input)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_shift_f32(_ptr(output), _ptr(input), delay * sign, n, T, Ts, stream),
                   "slayer_shift_f32")
    return output


def _delay_args(delay, x, n):
    """(table pointer, table size, scalar delay) of a delay given as a number, a one-element tensor
    or a tensor with one entry per neuron of a batch item."""
    if isinstance(delay, torch.Tensor):
        _check_input(delay, "delay")
        _check_device(x, delay, "input", "delay")
        if delay.numel() != 1:
            nBatch = x.shape[0]
            if nBatch == 0 or delay.numel() != n // nBatch:
                raise RuntimeError("shift and number of neurons must be same")
        return _ptr(delay), delay.numel(), 0.0
    return None, 0, _scalar(delay, "delay")


def getSpikesDelayed(d_u, d_nu, theta, Ts, delay, delayTs=1.0):
    """``shift(getSpikes(d_u, d_nu, theta, Ts), delay, delayTs)`` with the shift done while the spikes
    are stored (``d_u`` is updated in place and not shifted).  ``delay`` as in :func:`shift`.  Shapes
    the fused kernel does not serve run the two kernels."""
    _check_input(d_u, "d_u")
    _check_input(d_nu, "d_nu")
    _check_device(d_u, d_nu, "d_u", "d_nu")
    if d_u.dim() != 5:
        raise RuntimeError("getSpikesDelayed expects a 5 dimensional (N,C,H,W,T) tensor, got %d dimensions"
                           % d_u.dim())
    theta, Ts, delayTs = _scalar(theta, "theta"), _scalar(Ts, "Ts"), _scalar(delayTs, "delayTs")
    n, T = _rows(d_u)
    lut, lutSize, scalar = _delay_args(delay, d_u, n)
    lib = _lib.load()
    d_s = torch.empty_like(d_u)
    nuSize = d_nu.shape[-1] if d_nu.dim() else 1
    with _on_device_of(d_u) as stream:
        status = lib.slayer_get_spikes_delayed_f32(_ptr(d_s), _ptr(d_u), _ptr(d_nu), lut, lutSize, scalar, delayTs,
                                                   n, T, nuSize, theta, Ts, stream)
    if status == 2:      # not a shape of the fused kernel; nothing was launched
        return shift(getSpikes(d_u, d_nu, theta, Ts), delay, delayTs)
    _lib.check(status, "slayer_get_spikes_delayed_f32")
    return d_s


def spikeBackwardDelayed(gradOutput, membranePotential, theta, tau, scale, delay, delayTs=1.0):
    """``spikeBackward(shift(gradOutput, delay, delayTs, sign=-1), membranePotential, ...)`` in one
    pass: the backward of :func:`getSpikesDelayed` with respect to the membrane potential."""
    _check_input(gradOutput, "gradOutput")
    _check_input(membranePotential, "membranePotential")
    _check_device(gradOutput, membranePotential, "gradOutput", "membranePotential")
    if gradOutput.shape != membranePotential.shape:
        raise RuntimeError("gradOutput and membranePotential must have the same shape")
    theta, tau, scale = _scalar(theta, "theta"), _scalar(tau, "tau"), _scalar(scale, "scale")
    delayTs = _scalar(delayTs, "delayTs")
    n, T = _rows(gradOutput)
    lut, lutSize, scalar = _delay_args(delay, gradOutput, n)
    lib = _lib.load()
    gradInput = torch.empty_like(gradOutput)
    with _on_device_of(gradOutput) as stream:
        _lib.check(lib.slayer_spike_bwd_delayed_f32(_ptr(gradInput), _ptr(gradOutput), _ptr(membranePotential), lut,
                                                    lutSize, scalar, delayTs, n, T, theta, tau, scale, stream),
                   "slayer_spike_bwd_delayed_f32")
    return gradInput


def spikeBackward(gradOutput, membranePotential, theta, tau, scale):
    """``gradOutput * scale/tau * exp(-|membranePotential - theta| / tau)`` in one pass
    (``tau`` is the scaled time constant ``tauRho * theta``)."""
    _check_input(gradOutput, "gradOutput")
    _check_input(membranePotential, "membranePotential")
    _check_device(gradOutput, membranePotential, "gradOutput", "membranePotential")
    if gradOutput.shape != membranePotential.shape:
        raise RuntimeError("gradOutput and membranePotential must have the same shape")
    theta, tau, scale = _scalar(theta, "theta"), _scalar(tau, "tau"), _scalar(scale, "scale")
    lib = _lib.load()
    gradInput = torch.empty_like(gradOutput)
    with _on_device_of(gradOutput) as stream:
        _lib.check(lib.slayer_spike_bwd_f32(_ptr(gradInput), _ptr(gradOutput), _ptr(membranePotential),
                                            theta, tau, scale, gradOutput.numel(), stream),
                   "slayer_spike_bwd_f32")
    return gradInput


def pspSpike(input, srmKernel, refKernel, theta, Ts):
    """``conv(input, srmKernel, Ts)`` followed by ``getSpikes`` on the result, in one kernel where
    the shape allows (filters of 34 to 113 taps then run on the matrix cores, like ``conv`` on dense
    input).  Returns ``(spike, membranePotential)``; the membrane potential is the one after the
    refractory updates, as ``getSpikes`` leaves it."""
    _check_input(input, "input")
    _check_input(srmKernel, "srmKernel")
    _check_input(refKernel, "refKernel")
    _check_device(input, srmKernel, "input", "srmKernel")
    _check_device(input, refKernel, "input", "refKernel")
    if input.dim() != 5:
        raise RuntimeError("pspSpike expects a 5 dimensional (N,C,H,W,T) tensor, got %d dimensions" % input.dim())
    theta, Ts = _scalar(theta, "theta"), _scalar(Ts, "Ts")
    lib = _lib.load()
    spike = torch.empty_like(input)
    u = torch.empty_like(input)
    n, T = _rows(input)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_psp_spike_f32(_ptr(spike), _ptr(u), _ptr(input), _ptr(srmKernel), _ptr(refKernel),
                                            n, T, srmKernel.numel(), refKernel.numel(), theta, Ts, stream),
                   "slayer_psp_spike_f32")
    return spike, u


def spikeBackwardCorr(gradOutput, membranePotential, filter, theta, tau, scale, Ts):
    """``corr(spikeBackward(gradOutput, membranePotential, theta, tau, scale), filter, Ts)`` in one
    kernel, without the intermediate tensor (the backward pass of the Loihi neuron)."""
    _check_input(gradOutput, "gradOutput")
    _check_input(membranePotential, "membranePotential")
    _check_input(filter, "filter")
    _check_device(gradOutput, membranePotential, "gradOutput", "membranePotential")
    _check_device(gradOutput, filter, "gradOutput", "filter")
    if gradOutput.shape != membranePotential.shape:
        raise RuntimeError("gradOutput and membranePotential must have the same shape")
    theta, tau, scale, Ts = _scalar(theta, "theta"), _scalar(tau, "tau"), _scalar(scale, "scale"), _scalar(Ts, "Ts")
    lib = _lib.load()
    gradInput = torch.empty_like(gradOutput)
    nNeurons, T = _rows(gradOutput)
    with _on_device_of(gradOutput) as stream:
        _lib.check(lib.slayer_spike_bwd_corr_f32(_ptr(gradInput), _ptr(gradOutput), _ptr(membranePotential),
                                                 _ptr(filter), nNeurons, T, filter.numel(), theta, tau, scale, Ts,
                                                 stream),
                   "slayer_spike_bwd_corr_f32")
    return gradInput


def delayGrad(output, gradOutput, Ts):
    """Gradient of ``shift`` with respect to its per-neuron delays: ``Ts * sum over batch and
    time of gradOutput * (output[t-1] - output[t]) / Ts``; shape ``output.shape[1:-1]``."""
    _check_input(output, "output")
    _check_input(gradOutput, "gradOutput")
    _check_device(output, gradOutput, "output", "gradOutput")
    if output.shape != gradOutput.shape:
        raise RuntimeError("output and gradOutput must have the same shape")
    if output.dim() < 2:
        raise RuntimeError("delayGrad expects at least (batch, time) dimensions")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    T = output.shape[-1]
    nBatch = output.shape[0]
    shape = tuple(output.shape[1:-1])
    nPerBatch = 1
    for d in shape:
        nPerBatch *= d
    gradDelay = torch.empty(shape, dtype=output.dtype, device=output.device)
    nbytes = lib.slayer_delay_grad_workspace_bytes(nBatch, nPerBatch, T)
    workspace = torch.empty((max(nbytes, 4) // 4,), dtype=torch.float32, device=output.device)
    with _on_device_of(output) as stream:
        _lib.check(lib.slayer_delay_grad_f32(_ptr(gradDelay), _ptr(output), _ptr(gradOutput),
                                             workspace.data_ptr(), nBatch, nPerBatch, T, Ts, stream),
                   "slayer_delay_grad_f32")
    return gradDelay


def delayGradStatic(output, gradOutput, Ts, out=None):
    """``delayGrad`` without any device allocation inside the library call: the partial sums live in a
    fixed array of the library (at most ``slayer_delay_grad_static_max_rows()`` neuron rows), and the
    result goes into ``out`` when given (shape ``output.shape[1:-1]``).  For callers that must not
    allocate (graph capture, serving loops).  Calls that overlap on one GPU share the array and race."""
    _check_input(output, "output")
    _check_input(gradOutput, "gradOutput")
    _check_device(output, gradOutput, "output", "gradOutput")
    if output.shape != gradOutput.shape:
        raise RuntimeError("output and gradOutput must have the same shape")
    if output.dim() < 2:
        raise RuntimeError("delayGradStatic expects at least (batch, time) dimensions")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    T = output.shape[-1]
    nBatch = output.shape[0]
    shape = tuple(output.shape[1:-1])
    nPerBatch = 1
    for d in shape:
        nPerBatch *= d
    limit = lib.slayer_delay_grad_static_max_rows()
    if nBatch * nPerBatch > limit:
        raise RuntimeError("delayGradStatic serves at most %d neuron rows (got %d); use delayGrad"
                           % (limit, nBatch * nPerBatch))
    if out is None:
        out = torch.empty(shape, dtype=output.dtype, device=output.device)
    else:
        _check_input(out, "out")
        _check_device(output, out, "output", "out")
        if tuple(out.shape) != shape:
            raise RuntimeError("out must have shape %s" % (shape,))
    with _on_device_of(output) as stream:
        _lib.check(lib.slayer_delay_grad_static_f32(_ptr(out), _ptr(output), _ptr(gradOutput), nBatch, nPerBatch,
                                                    T, Ts, stream), "slayer_delay_grad_static_f32")
    return out


def spikeLoss(spikeOut, spikeDesired, srmKernel, Ts, addend=None):
    """``error = conv(spikeOut - spikeDesired, srmKernel, Ts) [+ addend]`` and
    ``loss = 1/2 * sum(error**2) * Ts`` in two launches.  Returns ``(loss, error)`` (``loss`` is a
    0-dim tensor), or ``None`` when a row does not fit the kernel (nothing was launched)."""
    _check_input(spikeOut, "spikeOut")
    _check_input(spikeDesired, "spikeDesired")
    _check_input(srmKernel, "srmKernel")
    _check_device(spikeOut, spikeDesired, "spikeOut", "spikeDesired")
    _check_device(spikeOut, srmKernel, "spikeOut", "srmKernel")
    if spikeOut.shape != spikeDesired.shape:
        raise RuntimeError("spikeOut and spikeDesired must have the same shape")
    if addend is not None:
        _check_input(addend, "addend")
        _check_device(spikeOut, addend, "spikeOut", "addend")
        if addend.shape != spikeOut.shape:
            raise RuntimeError("addend and spikeOut must have the same shape")
    Ts = _scalar(Ts, "Ts")
    lib = _lib.load()
    rows, T = _rows(spikeOut)
    loss = torch.empty((), dtype=spikeOut.dtype, device=spikeOut.device)
    error = torch.empty_like(spikeOut)
    workspace = torch.empty((max(rows, 1),), dtype=torch.float32, device=spikeOut.device)
    with _on_device_of(spikeOut) as stream:
        status = lib.slayer_spike_loss_f32(loss.data_ptr(), _ptr(error), _ptr(spikeOut), _ptr(spikeDesired),
                                           _ptr(addend) if addend is not None else None, _ptr(srmKernel),
                                           workspace.data_ptr(), rows, T, srmKernel.numel(), Ts, stream)
    if status == 2:
        return None
    _lib.check(status, "slayer_spike_loss_f32")
    return loss, error

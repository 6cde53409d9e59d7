"""Per-timestep synapses on (N, C, H, W, T) tensors over the C ABI of ``libslayer_hip.so``.

The reference's ``_convLayer`` / ``_poolLayer`` / ``_convTransposeLayer`` / ``_unpoolLayer`` call
``F.conv3d`` / ``F.conv_transpose3d`` with a kernel of time extent 1 (src/slayer.py:499-507,
:565-575, :631-643, :732-748) and leave the gradients to autograd.  Here the operation and its
two gradients are three extension-level functions on T-innermost tensors, tied together by
``synapseConv`` / ``synapseConvTranspose`` (autograd Functions with the argument meaning of the
torch calls they replace).  There is no CPU path: tensors must live on the GPU.
"""
import ctypes

import torch

from . import _lib
from .slayerCuda import _check_device, _check_input, _on_device_of, _ptr

__all__ = ["conv", "convGradInput", "convGradWeight", "outShape", "supported", "synapseConv", "synapseConvTranspose",
           "denseEvents", "denseEventsGradWeight", "denseEventsSupported", "synapseDenseEvents", "denseRows",
           "denseRowsSupported", "denseRowsPays", "synapseDenseRows", "denseRowsGradWeight",
           "denseRowsGradWeightSupported"]


def _pair(v, name):
    if isinstance(v, int):
        return v, v
    v = tuple(int(x) for x in v)
    if len(v) == 3 and name != "kernel":          # torch-style triple with the time entry last
        v = v[:2]
    if len(v) != 2:
        raise ValueError("%s must be an int or a pair, got %r" % (name, v))
    return v


def _geom(inShape, wShape, stride, padding, dilation, groups):
    if len(inShape) != 5:
        raise RuntimeError("expected a 5 dimensional (N,C,H,W,T) tensor, got %d dimensions" % len(inShape))
    if len(wShape) == 5:
        if wShape[4] != 1:
            raise RuntimeError("the synapse kernel must have a time extent of 1, got %d" % wShape[4])
        wShape = wShape[:4]
    if len(wShape) != 4:
        raise RuntimeError("expected a weight of shape (O, C/groups, KH, KW[, 1]), got %r" % (tuple(wShape),))
    N, C, H, W, T = (int(v) for v in inShape)
    O, Cg, KH, KW = (int(v) for v in wShape)
    groups = int(groups)
    if groups < 1 or C % groups or O % groups or Cg * groups != C:
        raise RuntimeError("weight of shape %r does not fit %d input channels in %d groups"
                           % (tuple(wShape), C, groups))
    (sH, sW), (pH, pW), (dH, dW) = _pair(stride, "stride"), _pair(padding, "padding"), _pair(dilation, "dilation")
    return _lib.SynapseGeom(N, C, H, W, T, O, KH, KW, sH, sW, pH, pW, dH, dW, groups)


def outShape(inShape, wShape, stride=1, padding=0, dilation=1, groups=1):
    """Shape (N, O, OH, OW, T) of ``conv`` for an input of shape ``inShape``."""
    g = _geom(inShape, wShape, stride, padding, dilation, groups)
    OH, OW = ctypes.c_int32(), ctypes.c_int32()
    _lib.check(_lib.load().slayer_synapse_out_shape(ctypes.byref(g), ctypes.byref(OH), ctypes.byref(OW)),
               "slayer_synapse_out_shape")
    return (g.N, g.O, OH.value, OW.value, g.T)


def supported(inShape, wShape, stride=1, padding=0, dilation=1, groups=1):
    """Whether the synapse kernels index this geometry: one batch item of the input and of the output below
    2 GiB, and a filter window - (padH + dilH * KH) rows plus (padW + dilW * KW) columns of the input - below
    16 MiB.  Decided on the host from the sizes alone (no GPU involved).  Beyond these limits the differentiable
    ``synapseConv`` / ``synapseConvTranspose`` fall back to torch's conv3d / conv_transpose3d, which the
    reference calls for every geometry."""
    g = _geom(inShape, wShape, stride, padding, dilation, groups)
    status = _lib.load().slayer_synapse_out_shape(ctypes.byref(g), None, None)
    if status == 2:
        return False
    _lib.check(status, "slayer_synapse_out_shape")
    return True


def _triple(v, last):
    a, b = _pair(v, "argument")
    return (a, b, last)


def conv(input, weight, stride=1, padding=0, dilation=1, groups=1):
    """``F.conv3d(input, weight, None, (sH,sW,1), (pH,pW,0), (dH,dW,1), groups)`` for a weight of
    time extent 1."""
    _check_input(input, "input")
    _check_input(weight, "weight")
    _check_device(input, weight, "input", "weight")
    g = _geom(input.shape, weight.shape, stride, padding, dilation, groups)
    lib = _lib.load()
    out = torch.empty(outShape(input.shape, weight.shape, stride, padding, dilation, groups),
                      dtype=input.dtype, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_synapse_conv_f32(_ptr(out), _ptr(input), _ptr(weight), ctypes.byref(g), stream),
                   "slayer_synapse_conv_f32")
    return out


def convGradInput(gradOutput, weight, inShape, stride=1, padding=0, dilation=1, groups=1):
    """Gradient of ``conv`` with respect to its input of shape ``inShape`` (= the transposed
    convolution of ``gradOutput``)."""
    _check_input(gradOutput, "gradOutput")
    _check_input(weight, "weight")
    _check_device(gradOutput, weight, "gradOutput", "weight")
    g = _geom(inShape, weight.shape, stride, padding, dilation, groups)
    expected = outShape(inShape, weight.shape, stride, padding, dilation, groups)
    if tuple(gradOutput.shape) != expected:
        raise RuntimeError("gradOutput has shape %r, expected %r" % (tuple(gradOutput.shape), expected))
    lib = _lib.load()
    gradIn = torch.empty(tuple(int(v) for v in inShape), dtype=gradOutput.dtype, device=gradOutput.device)
    with _on_device_of(gradOutput) as stream:
        _lib.check(lib.slayer_synapse_conv_grad_input_f32(_ptr(gradIn), _ptr(gradOutput), _ptr(weight),
                                                          ctypes.byref(g), stream),
                   "slayer_synapse_conv_grad_input_f32")
    return gradIn


def convGradWeight(gradOutput, input, wShape, stride=1, padding=0, dilation=1, groups=1):
    """Gradient of ``conv`` with respect to its weight of shape ``wShape``."""
    _check_input(gradOutput, "gradOutput")
    _check_input(input, "input")
    _check_device(gradOutput, input, "gradOutput", "input")
    g = _geom(input.shape, wShape, stride, padding, dilation, groups)
    expected = outShape(input.shape, wShape, stride, padding, dilation, groups)
    if tuple(gradOutput.shape) != expected:
        raise RuntimeError("gradOutput has shape %r, expected %r" % (tuple(gradOutput.shape), expected))
    lib = _lib.load()
    gradW = torch.empty(tuple(int(v) for v in wShape), dtype=input.dtype, device=input.device)
    nbytes = lib.slayer_synapse_conv_grad_weight_workspace_bytes(ctypes.byref(g))
    workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_synapse_conv_grad_weight_f32(_ptr(gradW), _ptr(gradOutput), _ptr(input),
                                                           _ptr(workspace), ctypes.byref(g), stream),
                   "slayer_synapse_conv_grad_weight_f32")
    return gradW


class _synapseConvFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation, groups):
        input = input.contiguous()
        weight = weight.contiguous()
        ctx.save_for_backward(input, weight)
        ctx.args = (stride, padding, dilation, groups)
        return conv(input, weight, *ctx.args)

    @staticmethod
    def backward(ctx, gradOutput):
        input, weight = ctx.saved_tensors
        gradOutput = gradOutput.contiguous()
        gradInput = gradWeight = None
        if ctx.needs_input_grad[0]:
            gradInput = convGradInput(gradOutput, weight, input.shape, *ctx.args)
        if ctx.needs_input_grad[1]:
            gradWeight = convGradWeight(gradOutput, input, weight.shape, *ctx.args)
        return gradInput, gradWeight, None, None, None, None


class _synapseConvTransposeFunction(torch.autograd.Function):
    """The transposed synapse: its forward pass is the input gradient of the convolution whose
    weight tensor it shares, its input gradient is that convolution."""

    @staticmethod
    def forward(ctx, input, weight, stride, padding, dilation, groups):
        input = input.contiguous()
        weight = weight.contiguous()
        (sH, sW), (pH, pW), (dH, dW) = _pair(stride, "stride"), _pair(padding, "padding"), _pair(dilation, "dilation")
        N, Cin, H, W, T = input.shape
        if weight.shape[0] != Cin:
            raise RuntimeError("weight of shape %r does not fit %d input channels" % (tuple(weight.shape), Cin))
        KH, KW = int(weight.shape[2]), int(weight.shape[3])
        outH = (H - 1) * sH - 2 * pH + dH * (KH - 1) + 1
        outW = (W - 1) * sW - 2 * pW + dW * (KW - 1) + 1
        ctx.outShape = (N, int(weight.shape[1]) * groups, outH, outW, T)
        ctx.save_for_backward(input, weight)
        ctx.args = (stride, padding, dilation, groups)
        return convGradInput(input, weight, ctx.outShape, *ctx.args)

    @staticmethod
    def backward(ctx, gradOutput):
        input, weight = ctx.saved_tensors
        gradOutput = gradOutput.contiguous()
        gradInput = gradWeight = None
        if ctx.needs_input_grad[0]:
            gradInput = conv(gradOutput, weight, *ctx.args)
        if ctx.needs_input_grad[1]:
            gradWeight = convGradWeight(input, gradOutput, weight.shape, *ctx.args)
        return gradInput, gradWeight, None, None, None, None


def synapseConv(input, weight, stride=1, padding=0, dilation=1, groups=1):
    """Differentiable ``conv``: stands where the reference calls ``F.conv3d(input, weight, None,
    stride, padding, dilation, groups)`` (src/slayer.py:499-507)."""
    if not supported(input.shape, weight.shape, stride, padding, dilation, groups):
        w5 = weight if weight.dim() == 5 else weight.unsqueeze(-1)
        return torch.nn.functional.conv3d(input, w5, None, _triple(stride, 1), _triple(padding, 0), _triple(dilation, 1),
                                          groups)
    return _synapseConvFunction.apply(input, weight, stride, padding, dilation, groups)


def synapseConvTranspose(input, weight, stride=1, padding=0, dilation=1, groups=1):
    """Differentiable transposed synapse: stands where the reference calls
    ``F.conv_transpose3d(input, weight, None, stride, padding, 0, groups, dilation)``
    (src/slayer.py:631-643)."""
    (sH, sW), (pH, pW), (dH, dW) = _pair(stride, "stride"), _pair(padding, "padding"), _pair(dilation, "dilation")
    KH, KW = int(weight.shape[2]), int(weight.shape[3])
    N, Cin, H, W, T = (int(v) for v in input.shape)
    # (the geometry of the convolution that this transposes: its input is this op's output)
    conv_in = (N, int(weight.shape[1]) * groups, (H - 1) * sH - 2 * pH + dH * (KH - 1) + 1,
               (W - 1) * sW - 2 * pW + dW * (KW - 1) + 1, T)
    if min(conv_in) >= 0 and not supported(conv_in, weight.shape[:4], stride, padding, dilation, groups):
        w5 = weight if weight.dim() == 5 else weight.unsqueeze(-1)
        return torch.nn.functional.conv_transpose3d(input, w5, None, _triple(stride, 1), _triple(padding, 0), 0, groups,
                                                    _triple(dilation, 1))
    return _synapseConvTransposeFunction.apply(input, weight, stride, padding, dilation, groups)


def denseEventsSupported(N, K, O, T):
    """Whether ``denseEvents`` and ``denseEventsGradWeight`` take these extents (the limits the header states)."""
    lim = (1 << 31) - 64
    return N <= 65535 and N * O * T * 4 < lim and O <= 1024 and K * O * 4 < lim and 0 < K and N * T < (1 << 22) \
        and T < (1 << 21)


def denseEvents(input, weight):
    """``weight @ input[n]`` for every batch item, ``input`` (N, K, T), ``weight`` (O, K), summed over the
    non-zero inputs only (ascending k): the dense layer's product for spike tensors.  The work grows with
    the number of non-zero inputs."""
    _check_input(input, "input")
    _check_input(weight, "weight")
    _check_device(input, weight, "input", "weight")
    if input.dim() != 3 or weight.dim() != 2 or weight.shape[1] != input.shape[1]:
        raise RuntimeError("denseEvents takes input (N, K, T) and weight (O, K); got %r and %r"
                           % (tuple(input.shape), tuple(weight.shape)))
    N, K, T = (int(v) for v in input.shape)
    O = int(weight.shape[0])
    lib = _lib.load()
    out = torch.empty((N, O, T), dtype=input.dtype, device=input.device)
    nbytes = lib.slayer_dense_events_workspace_bytes(N, K, O, T)
    workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_dense_events_f32(_ptr(out), _ptr(input), _ptr(weight), _ptr(workspace), N, K, O, T, stream),
                   "slayer_dense_events_f32")
    return out


def denseEventsGradWeight(gradOutput, input):
    """Weight gradient of the dense layer's product ``out[n] = weight @ input[n]``, ``input`` (N, K, T),
    ``gradOutput`` (N, O, T): ``sum_n gradOutput[n] @ input[n].T`` as (O, K), summed over the non-zero
    inputs only, in a fixed order.  The work grows with the number of non-zero inputs."""
    _check_input(gradOutput, "gradOutput")
    _check_input(input, "input")
    _check_device(gradOutput, input, "gradOutput", "input")
    if input.dim() != 3 or gradOutput.dim() != 3 or gradOutput.shape[0] != input.shape[0] \
            or gradOutput.shape[2] != input.shape[2]:
        raise RuntimeError("denseEventsGradWeight takes gradOutput (N, O, T) and input (N, K, T); got %r and %r"
                           % (tuple(gradOutput.shape), tuple(input.shape)))
    N, K, T = (int(v) for v in input.shape)
    O = int(gradOutput.shape[1])
    lib = _lib.load()
    gradW = torch.empty((O, K), dtype=input.dtype, device=input.device)
    nbytes = lib.slayer_dense_events_grad_weight_workspace_bytes(N, K, O, T)
    workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_dense_events_grad_weight_f32(_ptr(gradW), _ptr(gradOutput), _ptr(input), _ptr(workspace),
                                                           N, K, O, T, stream),
                   "slayer_dense_events_grad_weight_f32")
    return gradW


def denseRowsSupported(N, K, O, T):
    """Whether ``denseRows`` takes these extents (the limits the header states)."""
    return bool(_lib.load().slayer_dense_rows_supported(N, K, O, T))


def denseRows(input, weight, transposed=False):
    """``weight @ input[n]`` for every batch item, ``input`` (N, K, T), ``weight`` (O, K) - or, ``transposed``,
    ``weight.T @ input[n]`` with ``weight`` (K, O): the dense layer's product and its input gradient on bf16
    matrix instructions over split operands (``slayer_dense_rows_f32``), for layers with up to a few hundred
    inputs."""
    _check_input(input, "input")
    _check_input(weight, "weight")
    _check_device(input, weight, "input", "weight")
    if input.dim() != 3 or weight.dim() != 2 or weight.shape[0 if transposed else 1] != input.shape[1]:
        raise RuntimeError("denseRows takes input (N, K, T) and weight (O, K), or (K, O) transposed; got %r and %r"
                           % (tuple(input.shape), tuple(weight.shape)))
    N, K, T = (int(v) for v in input.shape)
    O = int(weight.shape[1 if transposed else 0])
    lib = _lib.load()
    out = torch.empty((N, O, T), dtype=input.dtype, device=input.device)
    wRow, wCol = (1, O) if transposed else (K, 1)
    workspace = torch.empty((lib.slayer_dense_rows_workspace_bytes(K, O) + 3) // 4, dtype=torch.float32, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_dense_rows_f32(_ptr(out), _ptr(weight), _ptr(input), _ptr(workspace), N, K, O, T, wRow, wCol,
                                             stream), "slayer_dense_rows_f32")
    return out


class _synapseDenseEventsFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight, product, gradient):
        ctx.save_for_backward(input, weight)
        ctx.gradient = gradient
        if product:
            return denseEvents(input, weight.contiguous())
        N, K, O = input.shape[0], input.shape[1], weight.shape[0]
        return torch.bmm(weight.unsqueeze(0).expand(N, O, K), input)

    @staticmethod
    def backward(ctx, gradOutput):
        input, weight = ctx.saved_tensors
        gradOutput = gradOutput.contiguous()
        gradInput = gradWeight = None
        if ctx.needs_input_grad[0]:   # the gradient is not sparse: a library product
            N, K, O = input.shape[0], input.shape[1], weight.shape[0]
            gradInput = torch.bmm(weight.t().unsqueeze(0).expand(N, K, O), gradOutput)
        if ctx.needs_input_grad[1]:
            if ctx.gradient:
                gradWeight = denseEventsGradWeight(gradOutput, input)
            else:
                gradWeight = torch.bmm(gradOutput, input.transpose(1, 2)).sum(0)
        return gradInput, gradWeight, None, None


def denseRowsGradWeightSupported(N, K, O, T):
    """Whether ``denseRowsGradWeight`` takes these extents (the limits the header states)."""
    return bool(_lib.load().slayer_dense_rows_grad_weight_supported(N, K, O, T))


def denseRowsGradWeight(gradOutput, input):
    """Weight gradient of the dense layer's product ``out[n] = weight @ input[n]``, ``input`` (N, K, T),
    ``gradOutput`` (N, O, T): ``sum_n gradOutput[n] @ input[n].T`` as (O, K), on bf16 matrix instructions over split
    operands (``slayer_dense_rows_grad_weight_f32``), for layers with up to 448 inputs and 256 outputs."""
    _check_input(gradOutput, "gradOutput")
    _check_input(input, "input")
    _check_device(gradOutput, input, "gradOutput", "input")
    if input.dim() != 3 or gradOutput.dim() != 3 or gradOutput.shape[0] != input.shape[0] \
            or gradOutput.shape[2] != input.shape[2]:
        raise RuntimeError("denseRowsGradWeight takes gradOutput (N, O, T) and input (N, K, T); got %r and %r"
                           % (tuple(gradOutput.shape), tuple(input.shape)))
    N, K, T = (int(v) for v in input.shape)
    O = int(gradOutput.shape[1])
    lib = _lib.load()
    gradW = torch.empty((O, K), dtype=input.dtype, device=input.device)
    nbytes = lib.slayer_dense_rows_grad_weight_workspace_bytes(N, K, O, T)
    workspace = torch.empty((nbytes + 3) // 4, dtype=torch.float32, device=input.device)
    with _on_device_of(input) as stream:
        _lib.check(lib.slayer_dense_rows_grad_weight_f32(_ptr(gradW), _ptr(gradOutput), _ptr(input), _ptr(workspace),
                                                         N, K, O, T, stream), "slayer_dense_rows_grad_weight_f32")
    return gradW


DENSE_ROWS_MAX_INPUTS = 448   # two launches of slayer_dense_rows_f32; beyond that the library product


def denseRowsPays(N, K, O, T):
    """Whether the dense layer's product (N, K, T) -> (N, O, T) is taken by ``denseRows``: few enough inputs, and enough
    work for a kernel that keeps the weights in registers (a library product is as fast on small problems)."""
    return K <= DENSE_ROWS_MAX_INPUTS and N * T >= 2048 and O >= 16 and denseRowsSupported(N, K, O, T)


def _aligned(t):
    """``t`` contiguous and on a 16-byte boundary (a view that starts inside an allocation is copied)."""
    t = t.contiguous()
    return t if t.data_ptr() % 16 == 0 else t.clone()


class _synapseDenseRowsFunction(torch.autograd.Function):
    @staticmethod
    def forward(ctx, input, weight):
        ctx.save_for_backward(input, weight)
        return denseRows(input, weight.contiguous())

    @staticmethod
    def backward(ctx, gradOutput):
        input, weight = ctx.saved_tensors
        gradOutput = _aligned(gradOutput)
        gradInput = gradWeight = None
        N, K, T = input.shape
        O = weight.shape[0]
        if ctx.needs_input_grad[0]:
            if denseRowsPays(N, O, K, T):     # (the outputs are what is summed over now)
                gradInput = denseRows(gradOutput, weight.contiguous(), transposed=True)
            else:
                gradInput = torch.bmm(weight.t().unsqueeze(0).expand(N, K, O), gradOutput)
        if ctx.needs_input_grad[1]:
            if N * T >= 2048 and denseRowsGradWeightSupported(N, K, O, T):
                gradWeight = denseRowsGradWeight(gradOutput, input)
            else:
                gradWeight = torch.bmm(gradOutput, input.transpose(1, 2)).sum(0)
        return gradInput, gradWeight


def synapseDenseRows(input, weight):
    """``weight @ input[n]`` for every batch item (``input`` (N, K, T), ``weight`` (O, K)) with its gradients, for
    layers with few inputs: product and input gradient from ``denseRows`` (bf16 matrix instructions over split
    operands, weights in registers), the weight gradient from ``denseRowsGradWeight`` (the library's batched product
    for more than 448 inputs or 256 outputs)."""
    return _synapseDenseRowsFunction.apply(_aligned(input), weight)


def synapseDenseEvents(input, weight, product=True, gradient=True):
    """``weight @ input[n]`` for every batch item (``input`` (N, K, T), ``weight`` (O, K)) with its gradients,
    for inputs that are spike tensors: the product (``product``) and the weight gradient (``gradient``) summed
    over the non-zero inputs (``denseEvents``, ``denseEventsGradWeight``) or as library matrix products; the
    input gradient - a product with the dense output gradient - always from the library."""
    return _synapseDenseEventsFunction.apply(input.contiguous(), weight, product, gradient)

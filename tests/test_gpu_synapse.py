"""Parity of the per-timestep synapse kernels (conv / pool / convTranspose / unpool layers and the
three C-ABI entry points behind them) with the CPU oracle on the same seeded inputs.

Tolerance: fp32 sums in a different order than the oracle's double accumulation, so every element
must satisfy |gpu - oracle| <= SUM_TOL * sum |terms| (the oracle evaluated on |x|, |w|), which is the
natural scale of a rounding error of a sum; for unit-scale data this is tighter than 1e-5 relative
to the largest output.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from _util import rel_err
from slayerpytorch_amd import _lib, synapse
import slayerpytorch_amd as snn

pytestmark = pytest.mark.gpu

SUM_TOL = 2e-6


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def close(got, ref, scale):
    assert got.shape == ref.shape
    err = np.abs(got.astype(np.float64) - ref)
    bound = SUM_TOL * scale + 1e-30
    worst = float((err / bound).max()) if err.size else 0.0
    assert worst <= 1.0, "error is %.2f x the bound" % worst


# (N, C, H, W, T, O, (KH, KW), stride, padding, dilation, groups)
CASES = [
    (2, 2, 9, 10, 12, 16, (5, 5), 1, 2, 1, 1),        # first CNN layer, small
    (1, 16, 7, 7, 8, 32, (3, 3), 1, 1, 1, 1),         # 144 taps
    (1, 32, 5, 5, 4, 20, (3, 3), 1, 1, 1, 1),         # 288 taps: two LDS chunks; 20 = 16 + 4 channels
    (2, 1, 12, 8, 16, 1, (2, 2), 2, 0, 1, 1),         # pooling geometry
    (1, 1, 13, 9, 8, 1, (3, 2), (3, 2), 0, 1, 1),     # ragged pooling: windows that do not fit
    (2, 1, 6, 8, 7, 1, (2, 2), 2, 0, 1, 1),           # pooling with T % 4 != 0
    (1, 1, 8, 8, 8, 1, (2, 2), 2, 1, 1, 1),           # padded pooling: overlapping the border, general kernel
    (2, 3, 8, 9, 7, 5, (3, 3), 1, 0, 1, 1),           # T % 4 != 0
    (1, 4, 10, 11, 6, 8, (3, 2), (2, 1), (1, 0), (1, 2), 2),   # stride, padding, dilation, groups
    (1, 6, 9, 9, 4, 6, (3, 3), 2, 2, 2, 3),           # all of them, 3 groups of 2
    (3, 5, 6, 6, 20, 3, (1, 1), 1, 0, 1, 1),          # 1x1
    (1, 2, 4, 4, 8, 2, (5, 5), 1, 0, 1, 1),           # filter larger than the input: empty output
    (1, 8, 6, 6, 4, 12, (2, 2), 1, 1, 1, 4),          # 3 output channels per group
    (2, 2, 34, 34, 300, 16, (5, 5), 1, 2, 1, 1),      # the benchmark's first layer on two samples
    # shapes that take the matrix-core weight gradient (T % 4 == 0, T >= 16, at least 8 tiles of 16 x 16)
    (1, 16, 7, 7, 32, 32, (3, 3), 1, 1, 1, 1),        # 2 x 9 tiles
    (1, 32, 5, 5, 20, 20, (3, 3), 1, 1, 1, 1),        # T % 16 != 0, 20 = 16 + 4 output channels, 18 column tiles
    (2, 32, 10, 11, 16, 48, (3, 2), (2, 1), (1, 0), (1, 2), 2),  # groups of 24 channels x 96 columns, stride, dilation
    (2, 15, 8, 9, 24, 9, (3, 3), 2, 1, 1, 1),         # stride 2, 9 output channels, 135 columns
    (1, 8, 6, 6, 64, 72, (3, 3), 1, 1, 1, 1),         # 72 output channels: two blocks of four tiles
    # ... with the input patch of four pixels staged in LDS per step of 32 samples: ragged pixel blocks (13 columns),
    # a last step of 12 samples, ranges of (block, step) pairs that cross batch items
    (3, 16, 9, 13, 44, 32, (3, 3), 1, 1, 1, 1),
    (2, 8, 6, 7, 100, 16, (5, 5), 1, 2, 1, 1),        # 200 columns: two column groups of 6 and 3 channels
    (2, 16, 6, 6, 36, 16, (3, 3), 1, 0, 2, 1),        # dilation 2 without padding: 2 x 2 output pixels
    # one or two destination channels and a filter at least 3 wide: four pixels of a row per lane
    (1, 8, 7, 9, 8, 2, (3, 3), 1, 1, 1, 1),           # forward with 2 output channels, 9 columns = 2 groups + 1 pixel
    (2, 1, 9, 11, 16, 8, (3, 5), 1, (1, 2), 1, 1),    # input gradient with 1 channel, 3 x 5 filter
    (1, 2, 10, 10, 8, 8, (3, 3), 1, (2, 1), (2, 1), 1),   # dilation along H only
    (1, 2, 6, 40, 4, 12, (1, 7), 1, (0, 3), 1, 1),    # 1 x 7 filter: 84 taps, 10 columns per lane
    # forward / input gradient on the matrix cores (at least 16 destination channels, passes of about 144 taps)
    (2, 32, 6, 9, 36, 64, (3, 3), 1, 1, 1, 1),        # two passes x two channel tiles; gradient: four passes
    (2, 32, 7, 10, 36, 32, (3, 3), 1, 1, 1, 2),       # two groups of 16 -> 16 channels, ranges crossing batch items
    (1, 4, 9, 9, 20, 16, (5, 5), 1, 2, 1, 1),         # 5 x 5: passes of 4 channels x 25 taps
    (1, 48, 5, 9, 32, 16, (3, 3), 1, 1, 1, 1),        # three passes; gradient: 48 channels = one and a half tile pairs
    (1, 12, 6, 8, 32, 16, (3, 4), 1, 1, 1, 1),        # 12 channels x 12 taps
    (1, 16, 8, 10, 64, 16, (3, 3), 1, (2, 1), (2, 1), 1),  # dilation along H
    (1, 16, 5, 8, 32, 20, (3, 3), 1, 1, 1, 1),        # 20 = 16 + 4 destination channels
]
IDS = ["%dx%dx%dx%dx%d-o%d-k%s-s%s-p%s-d%s-g%d" % c for c in CASES]


@pytest.fixture(params=[0, 1], ids=["fast", "generic"])
def impl(request):
    """Runs a test with the matrix-core / streaming kernels (default) and with the general vector
    kernels that serve every geometry."""
    lib = _lib.load()
    old = lib.slayer_force_generic_kernels(request.param)
    yield request.param
    lib.slayer_force_generic_kernels(old)


def make(case, seed):
    N, C, H, W, T, Oc, K, s, p, d, g = case
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((N, C, H, W, T)).astype(np.float32)
    w = rng.standard_normal((Oc, C // g, K[0], K[1])).astype(np.float32)
    return x, w, (s, p, d, g)


@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_conv_matches_oracle(case):
    x, w, a = make(case, 1)
    ref = O.synapse_conv(x, w, *a).astype(np.float64)
    got = host(synapse.conv(dev(x), dev(w), *a))
    close(got, ref, O.synapse_conv(np.abs(x), np.abs(w), *a))


@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_conv_grad_input_matches_oracle(case, impl):
    x, w, a = make(case, 2)
    shape = O.synapse_geom(x.shape, w.shape, *a)[1]
    go = np.random.default_rng(3).standard_normal(shape).astype(np.float32)
    ref = O.synapse_conv_grad_input(go, w, x.shape, *a).astype(np.float64)
    got = host(synapse.convGradInput(dev(go), dev(w), x.shape, *a))
    close(got, ref, O.synapse_conv_grad_input(np.abs(go), np.abs(w), x.shape, *a))


@pytest.mark.parametrize("case", CASES, ids=IDS)
def test_conv_grad_weight_matches_oracle(case, impl):
    x, w, a = make(case, 4)
    shape = O.synapse_geom(x.shape, w.shape, *a)[1]
    go = np.random.default_rng(5).standard_normal(shape).astype(np.float32)
    ref = O.synapse_conv_grad_weight(go, x, w.shape, *a).astype(np.float64)
    got = host(synapse.convGradWeight(dev(go), dev(x), w.shape, *a))
    close(got, ref, O.synapse_conv_grad_weight(np.abs(go), np.abs(x), w.shape, *a))


# the cases whose forward pass and weight gradient run bf16 matrix instructions
SPLIT_CASES = [c for c in CASES if c[5] >= 16 and (c[1] // c[10]) * c[6][0] * c[6][1] >= 96 and c[4] % 4 == 0 and c[4] >= 16]


@pytest.mark.parametrize("case", SPLIT_CASES, ids=["%dx%dx%dx%dx%d-o%d-k%s-s%s-p%s-d%s-g%d" % c for c in SPLIT_CASES])
@pytest.mark.parametrize("kind", ["spikes", "few bits", "one sample with all bits"])
def test_conv_and_grad_weight_on_inputs_that_are_bf16_numbers(case, kind):
    """Input samples with nothing below their upper 16 bits (spikes, small multiples of 1/8) take three of the six
    partial products; a single sample with more bits anywhere in a patch switches that patch to all six.  Forward
    pass and weight gradient against the oracle either way."""
    N, C, H, W, T, Oc, K, s_, p_, d_, g_ = case
    assert len(SPLIT_CASES) >= 8
    rng = np.random.default_rng(17)
    if kind == "spikes":
        x = (rng.random((N, C, H, W, T)) < 0.1).astype(np.float32)
    else:
        x = (rng.integers(-40, 41, (N, C, H, W, T)) / 8.0).astype(np.float32) * (rng.random((N, C, H, W, T)) < 0.5)
        x = x.astype(np.float32)
    if kind == "one sample with all bits":
        x[N - 1, C // 2, H // 2, W // 2, T // 3] = np.float32(np.pi)
    w = rng.standard_normal((Oc, C // g_, K[0], K[1])).astype(np.float32)
    a = (s_, p_, d_, g_)
    close(host(synapse.conv(dev(x), dev(w), *a)), O.synapse_conv(x, w, *a).astype(np.float64),
          O.synapse_conv(np.abs(x), np.abs(w), *a))
    shape = O.synapse_geom(x.shape, w.shape, *a)[1]
    go = rng.standard_normal(shape).astype(np.float32)
    close(host(synapse.convGradWeight(dev(go), dev(x), w.shape, *a)),
          O.synapse_conv_grad_weight(go, x, w.shape, *a).astype(np.float64),
          O.synapse_conv_grad_weight(np.abs(go), np.abs(x), w.shape, *a))


def test_random_geometries_against_conv3d():
    """60 seeded random layers with at least 16 output channels (the matrix-core kernels and what surrounds them: stride,
    padding, dilation, groups, ragged extents; spike inputs, dense inputs, inputs with few bits and one sample with all
    bits): forward pass and both gradients against torch's conv3d with a (KH, KW, 1) kernel and its autograd in
    double precision on the CPU, within SUM_TOL of the sum of the terms' magnitudes."""
    import torch.nn.functional as F
    rng = np.random.default_rng(321)
    done = 0
    while done < 60:
        g = int(rng.choice([1, 1, 1, 2]))
        Cg, Og = int(rng.choice([4, 8, 11, 12, 16, 16, 24, 32, 48])), int(rng.choice([16, 16, 20, 32, 33, 48, 64]))
        KH, KW = int(rng.choice([1, 2, 3, 3, 3, 5])), int(rng.choice([2, 3, 3, 3, 4, 5]))
        C, Oc = Cg * g, Og * g
        H, W = int(rng.integers(KH, 14)), int(rng.integers(KW, 20))
        T, N = 4 * int(rng.integers(4, 30)), int(rng.integers(1, 4))
        st = (int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2])))
        pd = (int(rng.integers(0, 3)), int(rng.integers(0, 3)))
        dl = (int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2])))
        if H + 2 * pd[0] - dl[0] * (KH - 1) - 1 < 0 or W + 2 * pd[1] - dl[1] * (KW - 1) - 1 < 0:
            continue
        kind = done % 3
        if kind == 0:
            x = (rng.random((N, C, H, W, T)) < 0.1).astype(np.float32)
        elif kind == 1:
            x = rng.standard_normal((N, C, H, W, T)).astype(np.float32)
        else:
            x = (rng.integers(-16, 17, (N, C, H, W, T)) / 4.0).astype(np.float32)
            x[0, 0, 0, 0, 0] = np.float32(0.1)
        w = rng.standard_normal((Oc, Cg, KH, KW)).astype(np.float32)

        def conv(xx, ww):
            return F.conv3d(xx, ww.unsqueeze(-1), None, st + (1,), pd + (0,), dl + (1,), g)
        xt, wt = torch.from_numpy(x).double().requires_grad_(True), torch.from_numpy(w).double().requires_grad_(True)
        y = conv(xt, wt)
        go = rng.standard_normal(tuple(y.shape)).astype(np.float32)
        y.backward(torch.from_numpy(go).double())
        xa, wa = xt.detach().abs().requires_grad_(True), wt.detach().abs().requires_grad_(True)
        ya = conv(xa, wa)
        ya.backward(torch.from_numpy(np.abs(go)).double())
        a = (st, pd, dl, g)
        what = "%s -> %d, %dx%d, %s" % ((N, C, H, W, T), Oc, KH, KW, a)
        for got, ref, scale in ((synapse.conv(dev(x), dev(w), *a), y, ya),
                                (synapse.convGradInput(dev(go), dev(w), x.shape, *a), xt.grad, xa.grad),
                                (synapse.convGradWeight(dev(go), dev(x), w.shape, *a), wt.grad, wa.grad)):
            err = (got.cpu().double() - ref.detach()).abs()
            assert bool((err <= SUM_TOL * scale.detach() + 1e-30).all()), what
        done += 1


def test_unaligned_storage():
    """Tensors that start 4 bytes into an allocation take the one-sample-per-lane kernels."""
    case = (1, 3, 6, 7, 8, 4, (3, 3), 1, 1, 1, 1)
    x, w, a = make(case, 6)
    shape = O.synapse_geom(x.shape, w.shape, *a)[1]
    go = np.random.default_rng(7).standard_normal(shape).astype(np.float32)

    def off(arr):
        buf = torch.empty(arr.size + 1, dtype=torch.float32, device="cuda")
        view = buf[1:].view(arr.shape)
        view.copy_(torch.from_numpy(arr))
        return view

    close(host(synapse.conv(off(x), dev(w), *a)), O.synapse_conv(x, w, *a).astype(np.float64),
          O.synapse_conv(np.abs(x), np.abs(w), *a))
    close(host(synapse.convGradInput(off(go), dev(w), x.shape, *a)),
          O.synapse_conv_grad_input(go, w, x.shape, *a).astype(np.float64),
          O.synapse_conv_grad_input(np.abs(go), np.abs(w), x.shape, *a))
    close(host(synapse.convGradWeight(off(go), off(x), w.shape, *a)),
          O.synapse_conv_grad_weight(go, x, w.shape, *a).astype(np.float64),
          O.synapse_conv_grad_weight(np.abs(go), np.abs(x), w.shape, *a))


def test_adjoint_identity_full_size():
    """<conv(x), g> == <x, gradInput(g)> == <w, gradWeight(g, x)> on the benchmark's first layer
    (12, 2, 34, 34, 300) -> 16 channels: a size-independent check of all three kernels."""
    gen = torch.Generator(device="cuda").manual_seed(0)
    x = (torch.rand((12, 2, 34, 34, 300), device="cuda", generator=gen) < 0.02).float()
    w = torch.randn((16, 2, 5, 5), device="cuda", generator=gen)
    y = synapse.conv(x, w, 1, 2)
    g = torch.randn(y.shape, device="cuda", generator=gen)
    lhs = float((y.double() * g.double()).sum())
    gi = synapse.convGradInput(g, w, x.shape, 1, 2)
    gw = synapse.convGradWeight(g, x, w.shape, 1, 2)
    scale = float((y.double().abs() * g.double().abs()).sum())
    assert abs(lhs - float((gi.double() * x.double()).sum())) <= 1e-6 * scale
    assert abs(lhs - float((gw.double() * w.double()).sum())) <= 1e-6 * scale


def test_argument_errors():
    lib = _lib.load()
    g = _lib.SynapseGeom(1, 4, 8, 8, 4, 6, 3, 3, 1, 1, 0, 0, 1, 1, 3)      # 4 channels in 3 groups
    assert lib.slayer_synapse_out_shape(g, None, None) == 1
    g = _lib.SynapseGeom(1, 4, 8, 8, 4, 6, 3, 3, 0, 1, 0, 0, 1, 1, 1)      # zero stride
    assert lib.slayer_synapse_conv_f32(None, None, None, g, None) == 1
    g = _lib.SynapseGeom(1, 4, 8, 8, 4, 6, 3, 3, 1, 1, 0, 0, 1, 1, 1)
    assert lib.slayer_synapse_conv_f32(None, None, None, g, None) == 1     # null pointers, non-empty output
    g = _lib.SynapseGeom(1, 64, 4096, 4096, 4, 6, 3, 3, 1, 1, 0, 0, 1, 1, 1)   # 4 GiB per batch item
    assert lib.slayer_synapse_out_shape(g, None, None) == 2
    with pytest.raises(RuntimeError):
        synapse.conv(torch.zeros((1, 4, 8, 8, 4), device="cuda"), torch.zeros((6, 3, 3, 3), device="cuda"))


# ---------------------------------------------------------------------------------------- layers
NEURON = {"type": "SRMALPHA", "theta": 10, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1,
          "scaleRho": 1}
SIM = {"Ts": 1.0, "tSample": 300}


def test_conv_layer_shift_and_add():
    """The construction of the reference's convolution test (test/test_slayer007.py:36-48)."""
    N, C, H, W, D, K = 2, 8, 20, 22, 24, 5
    layer = snn.layer(NEURON, SIM).cuda()
    conv = layer.conv(C, 1, K).cuda()
    x = torch.randn((N, C, H, W, D), device="cuda")
    weight = conv.weight.reshape(C, K, K)
    ref = torch.zeros((N, 1, H - K + 1, W - K + 1, D), device="cuda", dtype=torch.float64)
    for i in range(K):
        for j in range(K):
            for k in range(C):
                ref += weight[k, j, i].double() * x[:, k:k + 1, j:H - K + 1 + j, i:W - K + 1 + i, :].double()
    out = conv(x).detach()
    ref = ref.detach()
    assert float(torch.norm(out.double() - ref)) / out.numel() < 1e-6      # the reference's criterion
    assert float((out.double() - ref).abs().max()) <= 1e-5 * float(ref.abs().max())


def test_pool_layer_sum_of_four():
    """The construction of the reference's pooling test (test/test_slayer007.py:60-82), odd extents
    included."""
    layer = snn.layer(NEURON, SIM).cuda()
    pool = layer.pool(2).cuda()
    x = torch.randn((2, 3, 10, 12, 16), device="cuda")
    ref = (x[:, :, 0::2, 0::2] + x[:, :, 0::2, 1::2] + x[:, :, 1::2, 0::2] + x[:, :, 1::2, 1::2]) * 1.1 * NEURON["theta"]
    out = pool(x)
    assert out.shape == ref.shape
    assert float((out - ref).abs().max()) <= 1e-5 * float(ref.abs().max())
    odd = pool(torch.randn((2, 3, 11, 13, 8), device="cuda"))
    assert odd.shape == (2, 3, 6, 7, 8)


def test_conv_transpose_and_unpool_layers():
    """Transposed layers against their definition (test/test_slayer013.py): every input sample
    spreads its value, weighted, over the window it maps to."""
    layer = snn.layer(NEURON, SIM).cuda()
    Cin, C, K, H, W, D = 3, 4, 3, 6, 7, 8
    convT = layer.convTranspose(Cin, C, K).cuda()
    x = torch.randn((2, Cin, H, W, D), device="cuda")
    weight = convT.weight.reshape(Cin, C, K, K).double()
    ref = torch.zeros((2, C, H + K - 1, W + K - 1, D), device="cuda", dtype=torch.float64)
    for i in range(K):
        for j in range(K):
            for m in range(Cin):
                for k in range(C):
                    ref[:, k, i:i + H, j:j + W, :] += weight[m, k, i, j] * x[:, m].double()
    out = convT(x)
    assert out.shape == ref.shape
    assert float((out.double() - ref).abs().max()) <= 1e-5 * float(ref.abs().max())

    unpool = layer.unpool(2).cuda()
    x = torch.randn((2, 3, 5, 6, 8), device="cuda")
    out = unpool(x)
    ref = x.repeat_interleave(2, 2).repeat_interleave(2, 3) * 1.1 * NEURON["theta"]
    assert out.shape == ref.shape
    assert float((out - ref).abs().max()) <= 1e-5 * float(ref.abs().max())


@pytest.mark.parametrize("kind", ["conv", "pool", "convTranspose", "unpool"])
def test_layer_gradients_match_torch_cpu(kind):
    """Forward and both gradients of every synapse layer against the torch CPU op the reference's
    layer calls (F.conv3d / F.conv_transpose3d with a time extent of 1)."""
    import torch.nn.functional as F
    torch.manual_seed(11)
    layer = snn.layer(NEURON, SIM)
    if kind == "conv":
        mod = layer.conv(4, 6, 3, stride=1, padding=1, groups=2)
        x = torch.randn((2, 4, 7, 8, 12))
    elif kind == "pool":
        mod = layer.pool(2)
        x = torch.randn((2, 3, 8, 6, 12))
    elif kind == "convTranspose":
        mod = layer.convTranspose(4, 6, 3, stride=2, padding=1, groups=2)
        x = torch.randn((2, 4, 5, 6, 12))
    else:
        mod = layer.unpool(2)
        x = torch.randn((2, 3, 4, 5, 12))
    w = mod.weight.detach().clone()

    def torch_op(xc, wc):
        if kind == "conv":
            return F.conv3d(xc, wc, None, mod.stride, mod.padding, mod.dilation, mod.groups)
        if kind == "pool":
            s = xc.shape
            r = F.conv3d(xc.reshape(s[0], 1, s[1] * s[2], s[3], s[4]), wc, None, mod.stride, mod.padding, mod.dilation)
            return r.reshape(s[0], s[1], -1, r.shape[3], r.shape[4])
        if kind == "convTranspose":
            return F.conv_transpose3d(xc, wc, None, mod.stride, mod.padding, 0, mod.groups, mod.dilation)
        s = xc.shape
        r = F.conv_transpose3d(xc.reshape(s[0], 1, -1, s[3], s[4]), wc, None, mod.stride, mod.padding, 0, 1, mod.dilation)
        return r.reshape(s[0], s[1], -1, r.shape[3], r.shape[4])

    xc = x.clone().double().requires_grad_(True)
    wc = w.clone().double().requires_grad_(True)
    yc = torch_op(xc, wc)
    g = torch.randn(yc.shape)
    yc.backward(g.double())

    mod = mod.cuda()
    mod.weight.requires_grad_(True)
    xg = x.cuda().requires_grad_(True)
    yg = mod(xg)
    yg.backward(g.cuda())
    for got, ref in ((yg, yc), (xg.grad, xc.grad), (mod.weight.grad, wc.grad)):
        assert got.shape == ref.shape
        assert float((got.detach().cpu().double() - ref.detach()).abs().max()) <= 1e-5 * float(ref.abs().max())


# ------------------------------------------------------------------- dense layer, event by event
def dense_input(rng, shape, density, binary):
    x = (rng.random(shape) < density).astype(np.float32)
    if not binary:
        x *= rng.standard_normal(shape).astype(np.float32)
    return x


# (N, K, O, T, density, binary input)
DENSE_EVENT_CASES = [
    (2, 300, 37, 50, 0.05, True),          # ragged everything
    (1, 2312, 512, 64, 0.015, True),       # the NMNIST MLP's first layer: eight output channels per lane
    (3, 200, 256, 130, 0.04, False),       # T % 4 != 0, real-valued events
    (2, 600, 10, 33, 1.0, False),          # nothing to skip
    (2, 64, 700, 48, 0.1, True),           # 11 output channels per lane
    (5, 40, 1024, 70, 0.2, True),          # the most output channels; five blocks: one group of four and one more
    (4, 7, 3, 5, 0.5, False),              # tiny
    (2, 513, 65, 16, 0.0, True),           # no events at all
]


@pytest.mark.parametrize("case", DENSE_EVENT_CASES)
def test_dense_events_product_and_weight_gradient(case):
    N, K, O, T, density, binary = case
    rng = np.random.default_rng(N + K + O + T)
    x = dense_input(rng, (N, K, T), density, binary)
    x[0, 0, : min(T, 3)] = -0.0                               # a negative zero is no event
    w = rng.standard_normal((O, K)).astype(np.float32)
    ref = np.einsum("ok,nkt->not", w.astype(np.float64), x.astype(np.float64))
    scale = np.einsum("ok,nkt->not", np.abs(w).astype(np.float64), np.abs(x).astype(np.float64))
    got = synapse.denseEvents(dev(x), dev(w))
    close(host(got), ref, scale)
    assert torch.equal(got, synapse.denseEvents(dev(x), dev(w)))                 # fixed order of the additions
    if density == 0.0:
        assert not host(got).any()
    g = rng.standard_normal((N, O, T)).astype(np.float32)
    refW = np.einsum("not,nkt->ok", g.astype(np.float64), x.astype(np.float64))
    scaleW = np.einsum("not,nkt->ok", np.abs(g).astype(np.float64), np.abs(x).astype(np.float64))
    gotW = synapse.denseEventsGradWeight(dev(g), dev(x))
    close(host(gotW), refW, scaleW)
    assert torch.equal(gotW, synapse.denseEventsGradWeight(dev(g), dev(x)))      # fixed order of the additions
    if density == 0.0:
        assert not host(gotW).any()


def test_dense_events_weight_gradient_in_slices():
    # few input channels and many samples: the batch's samples are cut into slices that are added up afterwards
    lib = _lib.load()
    N, K, O, T = 16, 12, 20, 2000
    assert lib.slayer_dense_events_grad_weight_workspace_bytes(N, K, O, T) > (N * T * O + K * O) * 4   # more than one slice
    assert lib.slayer_dense_events_grad_weight_workspace_bytes(0, K, O, T) == 0
    rng = np.random.default_rng(5)
    x = dense_input(rng, (N, K, T), 0.03, True)
    g = rng.standard_normal((N, O, T)).astype(np.float32)
    refW = np.einsum("not,nkt->ok", g.astype(np.float64), x.astype(np.float64))
    scaleW = np.einsum("not,nkt->ok", np.abs(g).astype(np.float64), np.abs(x).astype(np.float64))
    close(host(synapse.denseEventsGradWeight(dev(g), dev(x))), refW, scaleW)


def test_dense_events_status_codes():
    lib = _lib.load()
    t = torch.full((64,), 7.0, device="cuda")
    p = t.data_ptr()
    assert lib.slayer_dense_events_f32(None, None, None, None, 0, 5, 5, 8, None) == 0                 # empty: nothing to do
    u = torch.full((64,), 7.0, device="cuda")
    assert lib.slayer_dense_events_f32(u.data_ptr(), None, None, None, 2, 0, 3, 5, None) == 0         # no inputs: zeros
    torch.cuda.synchronize()
    assert not u[:30].any() and bool((u[30:] == 7.0).all())
    assert lib.slayer_dense_events_f32(None, p, p, p, 1, 5, 5, 8, None) == 1
    assert lib.slayer_dense_events_f32(p, p, p, None, 1, 5, 5, 8, None) == 1
    assert lib.slayer_dense_events_f32(p, p, p, p, 1, 5, 1025, 8, None) == 2
    assert lib.slayer_dense_events_f32(p, p, p, p, 65536, 5, 5, 8, None) == 2
    assert lib.slayer_dense_events_f32(p, p, p, p, 1, 1 << 20, 1024, 8, None) == 2                    # weights over 2 GiB
    assert lib.slayer_dense_events_workspace_bytes(0, 5, 5, 8) == 0
    assert lib.slayer_dense_events_grad_weight_f32(None, None, None, None, 1, 0, 5, 8, None) == 0     # no weights: nothing to do
    assert lib.slayer_dense_events_grad_weight_f32(p, None, None, None, 0, 5, 5, 8, None) == 0        # no samples: zeros
    torch.cuda.synchronize()
    assert not t[:25].any() and bool((t[25:] == 7.0).all())
    assert lib.slayer_dense_events_grad_weight_f32(p, p, p, p, 1, 5, 1025, 8, None) == 2
    assert lib.slayer_dense_events_grad_weight_f32(p, p, p, p, 2, 5, 1024, 1 << 18, None) == 2         # gradOut of 2 GiB
    assert lib.slayer_dense_events_grad_weight_f32(p, p, p, p, 65536, 5, 5, 8, None) == 2
    assert lib.slayer_dense_events_grad_weight_f32(None, p, p, p, 1, 5, 5, 8, None) == 1
    assert lib.slayer_dense_events_grad_weight_f32(p, None, p, p, 1, 5, 5, 8, None) == 1
    assert lib.slayer_dense_events_grad_weight_f32(p, p, p, None, 1, 5, 5, 8, None) == 1
    assert lib.slayer_dense_events_grad_weight_f32(p, p, p, p, -1, 5, 5, 8, None) == 1
    with pytest.raises(_lib.SlayerHipError, match="not supported"):
        synapse.denseEventsGradWeight(torch.zeros((1, 1025, 8), device="cuda"), torch.zeros((1, 5, 8), device="cuda"))


# (N, K, O, T, spike input)
DENSE_ROWS_CASES = [
    (2, 200, 256, 64, True),       # the long-sequence network's first layer: seven chunks of inputs, all eight wavefronts
    (2, 200, 256, 64, False),      # the same on a dense input: all six products
    (3, 7, 5, 36, False),          # tiny: one chunk, one wavefront at work, a tile of 4 samples at the end
    (2, 256, 200, 100, True),      # more than 224 inputs: two launches that add up; 200 outputs: a wavefront with 8 rows
    (2, 300, 40, 2000, False),     # long rows: many tiles per work-group
    (1, 32, 16, 4, False),         # a single tile of four samples
    (2, 224, 300, 96, True),       # more than 256 outputs: two groups of wavefronts
    (1, 448, 33, 68, False),       # the most inputs the layer sends here
    (70, 96, 64, 32, True),        # more tiles than one per batch item... one tile each, 70 items
]


@pytest.mark.parametrize("case", DENSE_ROWS_CASES)
@pytest.mark.parametrize("transposed", [False, True])
def test_dense_rows_product(case, transposed):
    # the dense layer's product and (transposed) input gradient on bf16 matrix instructions over split operands: every
    # output within 1e-6 of the sum of its terms' magnitudes (the bound the header states; the north star asks for
    # 1e-5), on spikes and on dense inputs of mixed magnitude
    N, K, O, T, spikes = case
    rng = np.random.default_rng(N + K + O + T)
    x = dense_input(rng, (N, K, T), 0.04, True) if spikes else \
        (rng.standard_normal((N, K, T)) * np.exp2(rng.integers(-8, 8, (N, K, T)))).astype(np.float32)
    w = (rng.standard_normal((K, O) if transposed else (O, K)) * np.exp2(rng.integers(-6, 6, (K, O) if transposed else (O, K)))).astype(np.float32)
    W = (w.T if transposed else w).astype(np.float64)
    ref = np.einsum("ok,nkt->not", W, x.astype(np.float64))
    scale = np.einsum("ok,nkt->not", np.abs(W), np.abs(x).astype(np.float64))
    got = synapse.denseRows(dev(x), dev(w), transposed)
    err = np.abs(host(got).astype(np.float64) - ref)
    assert np.all(err <= 1e-6 * scale + 1e-30), float((err / (scale + 1e-30)).max())
    assert torch.equal(got, synapse.denseRows(dev(x), dev(w), transposed))            # the same bits every time


# (N, K, O, T, spike input)
DENSE_ROWS_GRAD_WEIGHT_CASES = [
    (2, 24, 20, 64, False),        # two tiles of inputs, one wavefront at work
    (3, 200, 256, 300, False),     # the long-sequence network: 13 tiles of inputs, all wavefronts, a chunk of 12 samples at the end
    (5, 37, 70, 124, True),        # sizes that divide by nothing: a sum row that is not a multiple of four long
    (2, 208, 256, 96, True),       # the most inputs of one launch
    (2, 256, 200, 100, True),      # two blocks of 128 inputs; 200 outputs: a wavefront with 8 rows
    (2, 448, 30, 100, False),      # the most inputs: three blocks
    (70, 16, 250, 32, True),       # one chunk per item, more items than one per work-group... 70 chunks
    (1, 16, 16, 4, False),         # a single chunk of four samples
    (6, 128, 128, 3000, True),     # long rows: more chunks than work-groups, several per group
]


@pytest.mark.parametrize("case", DENSE_ROWS_GRAD_WEIGHT_CASES)
def test_dense_rows_grad_weight(case):
    # the dense layer's weight gradient on bf16 matrix instructions over split operands: every element within 1e-6 of
    # the sum of its terms' magnitudes (the bound the header states), on spikes and on dense inputs of mixed magnitude
    N, K, O, T, spikes = case
    rng = np.random.default_rng(N + K + O + T)
    x = dense_input(rng, (N, K, T), 0.04, True) if spikes else \
        (rng.standard_normal((N, K, T)) * np.exp2(rng.integers(-8, 8, (N, K, T)))).astype(np.float32)
    g = (rng.standard_normal((N, O, T)) * np.exp2(rng.integers(-6, 6, (N, O, T)))).astype(np.float32)
    ref = np.einsum("not,nkt->ok", g.astype(np.float64), x.astype(np.float64))
    scale = np.einsum("not,nkt->ok", np.abs(g).astype(np.float64), np.abs(x).astype(np.float64))
    got = synapse.denseRowsGradWeight(dev(g), dev(x))
    assert got.shape == (O, K)
    err = np.abs(host(got).astype(np.float64) - ref)
    assert np.all(err <= 1e-6 * scale + 1e-30), float((err / (scale + 1e-30)).max())
    assert torch.equal(got, synapse.denseRowsGradWeight(dev(g), dev(x)))                # the same bits every time


def test_dense_rows_grad_weight_status_codes_and_limits():
    lib = _lib.load()
    t = torch.full((4096,), 7.0, device="cuda")
    p = t.data_ptr()
    fn = lib.slayer_dense_rows_grad_weight_f32
    assert fn(None, None, None, None, 1, 0, 5, 8, None) == 0                              # no weights: nothing to do
    assert fn(None, p, p, p, 1, 5, 5, 8, None) == 1
    assert fn(p, p, p, None, 1, 5, 5, 8, None) == 1
    assert fn(p, p, p, p, 1, 5, 5, 6, None) == 2                                          # T % 4 != 0
    assert fn(p, p + 4, p, p, 1, 5, 5, 8, None) == 2                                      # gradOut not 16-byte aligned
    assert fn(p, p, p, p, 1, 449, 5, 8, None) == 2 and fn(p, p, p, p, 1, 5, 257, 8, None) == 2
    assert fn(p + 4, None, None, None, 0, 3, 5, 8, None) == 0                             # an empty batch: zeros
    torch.cuda.synchronize()
    assert host(t[1:16]).tolist() == [0.0] * 15 and host(t[16:18]).tolist() == [7.0, 7.0] and float(t[0]) == 7.0
    assert not synapse.denseRowsGradWeightSupported(1, 5, 5, 6) and synapse.denseRowsGradWeightSupported(1, 448, 256, 8)
    assert lib.slayer_dense_rows_grad_weight_workspace_bytes(0, 5, 5, 8) == 0
    # one row of sums (padded to a multiple of four) for each of the 2 x 3 chunks
    assert lib.slayer_dense_rows_grad_weight_workspace_bytes(2, 5, 5, 68) == 6 * 28 * 4
    with pytest.raises(RuntimeError, match="denseRowsGradWeight takes"):
        synapse.denseRowsGradWeight(torch.zeros((1, 5, 8), device="cuda"), torch.zeros((2, 4, 8), device="cuda"))


def test_dense_rows_kernels_on_random_shapes():
    """120 seeded random shapes (1-448 inputs, 1-299 outputs, the limits of a launch and of a block among them; spikes and
    dense inputs of mixed magnitude): product, input gradient and weight gradient within 1e-6 of the sum of the
    terms' magnitudes."""
    rng = np.random.default_rng(123)
    for it in range(120):
        N, K, Oc, T = int(rng.integers(1, 6)), int(rng.integers(1, 449)), int(rng.integers(1, 300)), 4 * int(rng.integers(1, 80))
        if it % 7 == 0:
            K = int(rng.choice([1, 31, 32, 33, 208, 209, 224, 225, 416, 448]))
        if it % 11 == 0:
            Oc = int(rng.choice([1, 15, 16, 17, 255, 256, 257, 290]))
        x = (rng.random((N, K, T)) < 0.1).astype(np.float32) if it % 2 else \
            (rng.standard_normal((N, K, T)) * np.exp2(rng.integers(-6, 6, (N, K, T)))).astype(np.float32)
        w = rng.standard_normal((Oc, K)).astype(np.float32)
        g = rng.standard_normal((N, Oc, T)).astype(np.float32)
        x64, w64, g64 = x.astype(np.float64), w.astype(np.float64), g.astype(np.float64)
        checks = [(synapse.denseRows(dev(x), dev(w)), "ok,nkt->not", (w64, x64)),
                  (synapse.denseRows(dev(g), dev(w), transposed=True), "ok,not->nkt", (w64, g64))]
        if synapse.denseRowsGradWeightSupported(N, K, Oc, T):
            checks.append((synapse.denseRowsGradWeight(dev(g), dev(x)), "not,nkt->ok", (g64, x64)))
        for got, spec, ops in checks:
            ref = np.einsum(spec, *ops)
            scale = np.einsum(spec, *[np.abs(o) for o in ops])
            err = np.abs(host(got).astype(np.float64) - ref)
            assert np.all(err <= 1e-6 * scale + 1e-30), (N, K, Oc, T, spec, float((err / (scale + 1e-30)).max()))


def test_dense_rows_status_codes_and_limits():
    lib = _lib.load()
    t = torch.full((4096,), 7.0, device="cuda")
    p = t.data_ptr()
    assert lib.slayer_dense_rows_f32(None, None, None, None, 0, 5, 5, 8, 5, 1, None) == 0                 # empty: nothing to do
    assert lib.slayer_dense_rows_f32(None, p, p, p, 1, 5, 5, 8, 5, 1, None) == 1
    assert lib.slayer_dense_rows_f32(p, p, p, None, 1, 5, 5, 8, 5, 1, None) == 1
    assert lib.slayer_dense_rows_f32(p, p, p, p, 1, 5, 5, 6, 5, 1, None) == 2                             # T % 4 != 0
    assert lib.slayer_dense_rows_f32(p, p, p + 4, p, 1, 5, 5, 8, 5, 1, None) == 2                         # x not 16-byte aligned
    assert lib.slayer_dense_rows_f32(p, p, p, p, 1, 5, 5, 1 << 30, 5, 1, None) == 2                       # rows over 2 GiB
    assert not lib.slayer_dense_rows_supported(1, 5, 5, 6) and lib.slayer_dense_rows_supported(1, 5, 5, 8)
    assert lib.slayer_dense_rows_workspace_bytes(0, 5) == 0
    # eight wavefronts x two halves x seven chunks x three parts of 1 KiB
    assert lib.slayer_dense_rows_workspace_bytes(200, 256) == 8 * 2 * 7 * 3 * 1024
    assert synapse.denseRowsPays(64, 200, 256, 2000) and not synapse.denseRowsPays(64, 449, 256, 2000)
    assert not synapse.denseRowsPays(64, 200, 256, 2001) and not synapse.denseRowsPays(1, 200, 256, 64)
    with pytest.raises(RuntimeError, match="denseRows takes"):
        synapse.denseRows(torch.zeros((1, 5, 8), device="cuda"), torch.zeros((4, 6), device="cuda"))


def test_dense_layer_with_few_inputs_runs_dense_rows(monkeypatch):
    """_denseLayer with 200 inputs: product and both gradients from synapse.denseRows*, against the library products
    (DENSE_ROWS = False): outputs and all gradients to rounding."""
    from slayerpytorch_amd import slayer as slayer_module
    params = {"type": "SRMALPHA", "theta": 10, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    T = 512
    layer = snn.layer(params, {"Ts": 1.0, "tSample": T}).cuda()
    torch.manual_seed(5)
    fc = layer.dense(200, 96).cuda()
    rng = np.random.default_rng(11)
    g = dev(rng.standard_normal((4, 96, 1, 1, T)).astype(np.float32))
    calls = []
    real = synapse.denseRows
    monkeypatch.setattr(synapse, "denseRows", lambda *a, **k: (calls.append(1), real(*a, **k))[1])
    realGrad, gradCalls = synapse.denseRowsGradWeight, []
    monkeypatch.setattr(synapse, "denseRowsGradWeight", lambda *a, **k: (gradCalls.append(1), realGrad(*a, **k))[1])
    for x0 in (dense_input(rng, (4, 200, 1, 1, T), 0.03, True), rng.standard_normal((4, 200, 1, 1, T)).astype(np.float32)):
        results = []
        for mode in (True, False):
            monkeypatch.setattr(slayer_module, "DENSE_ROWS", mode)
            x = dev(x0).requires_grad_(True)
            fc.weight.grad = None
            n, m = len(calls), len(gradCalls)
            y = fc(x)
            y.backward(g)
            assert (len(calls) - n) == (2 if mode else 0)        # the product and the input gradient
            assert (len(gradCalls) - m) == (1 if mode else 0)    # the weight gradient
            results.append((host(y), host(x.grad), host(fc.weight.grad)))
        for a, b in zip(*results):
            assert rel_err(a, b) <= 1e-5


def test_dense_rows_layer_on_a_view_that_is_not_16_byte_aligned():
    """synapseDenseRows copies an input (or an output gradient) that starts 4 bytes into an allocation; same values as
    on an aligned tensor."""
    rng = np.random.default_rng(23)
    N, K, O, T = 2, 40, 32, 1024
    x = rng.standard_normal((N, K, T)).astype(np.float32)
    g = rng.standard_normal((N, O, T)).astype(np.float32)
    w = dev(rng.standard_normal((O, K)).astype(np.float32))

    def off(arr):
        buf = torch.empty(arr.size + 1, dtype=torch.float32, device="cuda")
        view = buf[1:].view(arr.shape)
        view.copy_(torch.from_numpy(arr))
        return view

    results = []
    for place in (dev, off):
        xi = place(x).requires_grad_(True)
        wi = w.clone().requires_grad_(True)
        y = synapse.synapseDenseRows(xi, wi)
        y.backward(place(g))
        results.append((host(y), host(xi.grad), host(wi.grad)))
    assert off(x).data_ptr() % 16 != 0
    for a, b in zip(*results):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("shape", [((34, 34, 2), 40, 12), (50, 10, 33)])
def test_dense_layer_sums_over_the_events_of_sparse_input(shape, monkeypatch):
    """_denseLayer with the event-driven product and weight gradient against the library products: same output and
    gradients to rounding (the input gradient is the library's either way); left to itself the layer measures
    its input and picks the events for spike tensors with many channels only."""
    from slayerpytorch_amd import slayer as slayer_module
    inFeatures, O, T = shape
    params = {"type": "SRMALPHA", "theta": 10, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    layer = snn.layer(params, {"Ts": 1.0, "tSample": T}).cuda()
    torch.manual_seed(3)
    fc = layer.dense(inFeatures, O).cuda()
    C, H, W = fc.weight.shape[1:4]
    rng = np.random.default_rng(9)
    x = dense_input(rng, (3, C, H, W, T), 0.02, True)
    g = dev(rng.standard_normal((3, O, 1, 1, T)).astype(np.float32))
    results = []
    for mode in (True, False):
        monkeypatch.setattr(slayer_module, "DENSE_EVENTS", mode)
        xt = dev(x).requires_grad_(True)
        fc.weight.grad = None
        y = fc(xt)
        y.backward(g)
        results.append((y.detach(), xt.grad.clone(), fc.weight.grad.clone()))
    assert torch.equal(results[0][1], results[1][1])
    K = C * H * W
    w2 = host(fc.weight).reshape(O, K).astype(np.float64)
    x3 = x.reshape(3, K, T).astype(np.float64)
    g3 = host(g).reshape(3, O, T).astype(np.float64)
    for y, gx, gw in results:
        close(host(y).reshape(3, O, T), np.einsum("ok,nkt->not", w2, x3), np.einsum("ok,nkt->not", np.abs(w2), np.abs(x3)))
        close(host(gx).reshape(3, K, T), np.einsum("ok,not->nkt", w2, g3), np.einsum("ok,not->nkt", np.abs(w2), np.abs(g3)))
        close(host(gw).reshape(O, K), np.einsum("not,nkt->ok", g3, x3), np.einsum("not,nkt->ok", np.abs(g3), np.abs(x3)))
    monkeypatch.setattr(slayer_module, "DENSE_EVENTS", "auto")
    fc(dev(x))
    many = K >= slayer_module.DENSE_EVENTS_MIN_CHANNELS
    assert fc._inputIsSparse(dev(x).reshape(3, K, T)) == ((True, True) if many else (False, False))
    assert (abs(fc._eventDensity - float((x != 0).mean())) < 1e-6) if many else fc._eventDensity is None
    other = layer.dense(inFeatures, O).cuda()
    other(dev(rng.standard_normal((3, C, H, W, T)).astype(np.float32)))
    assert other._inputIsSparse(dev(x).reshape(3, K, T)) == (False, False)      # (the measurement of the last call decides)
    # in between: the weight gradient alone
    third = layer.dense(inFeatures, O).cuda()
    mid = dense_input(rng, (3, C, H, W, T), 0.04, True)
    third(dev(mid))
    assert third._inputIsSparse(dev(mid).reshape(3, K, T)) == ((False, True) if many else (False, False))
    with torch.no_grad():                                          # inference takes the events as well
        close(host(fc(dev(x))).reshape(3, O, T), np.einsum("ok,nkt->not", w2, x3), np.einsum("ok,nkt->not", np.abs(w2), np.abs(x3)))

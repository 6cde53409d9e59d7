"""Whole networks on the GPU: a training loop over many optimiser steps (the analogue of the reference's
test/test_slayer005.py:79-94 on its 250-25-1 fixture), the host-side state that only shows over many steps
(pairing notes, kernel stamps, the dense layer's density measurement), ``utils.capturedStep``, and one training
step of the NMNIST-shaped MLP and of the CNN's first layers at their full batch size against the CPU oracle chain.
"""
import io

import numpy as np
import pytest
import torch

import slayerpytorch_amd as snn
from oracle import oracle as O
from slayerpytorch_amd import slayer as slayer_module
from slayerpytorch_amd.utils import capturedStep

from _util import golden, raster_from_aer, rel_err

pytestmark = pytest.mark.gpu

DEV = "cuda"


def neuron(**kw):
    d = {"theta": 10.0, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2.0, "tauRho": 1.0, "scaleRho": 1.0}
    d.update(kw)
    return d


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    return t.detach().cpu().numpy()


# ------------------------------------------------------------------------- many optimiser steps
def train_golden_network(steps, monkeypatch, switches):
    """Adam on the 250-25-1 network of the reference's fixture (test/test_slayer005.py:26-94: forward
    spike(fc(psp(.))) twice, spike-time loss, Adam lr 0.01 amsgrad); returns the losses, the allocated bytes after
    every step and the final weights."""
    for name, value in switches.items():
        monkeypatch.setattr(slayer_module, name, value)
    snn_d = golden("snn_250_25_1.npz")
    Ts, Ns = 0.1, 500
    nd = neuron(tauSr=1.0, tauRho=0.1)
    sim = {"Ts": Ts, "tSample": 50}
    layer = snn.layer(nd, sim).to(DEV)
    fc1, fc2 = layer.dense(250, 25).to(DEV), layer.dense(25, 1).to(DEV)
    fc1.weight = torch.nn.Parameter(dev(snn_d["w1Initial"]).reshape(25, 250, 1, 1, 1))
    fc2.weight = torch.nn.Parameter(dev(snn_d["w2Initial"]).reshape(1, 25, 1, 1, 1))
    x = dev(raster_from_aer(snn_d["spikeIn"], 250, Ns, Ts, 1 / Ts)).reshape(1, 250, 1, 1, Ns)
    des = dev(raster_from_aer(snn_d["spikeOut"], 1, Ns, Ts, 1 / Ts)).reshape(1, 1, 1, 1, Ns)
    error = snn.loss({"neuron": nd, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}).to(DEV)
    optimizer = torch.optim.Adam([fc1.weight, fc2.weight], lr=0.01, amsgrad=True)
    losses, allocated = [], []
    for _ in range(steps):
        s1 = layer.spike(fc1(layer.psp(x)))
        s2 = layer.spike(fc2(layer.psp(s1)))
        loss = error.spikeTime(s2, des)
        losses.append(float(loss.detach()))
        optimizer.zero_grad()
        loss.backward()
        optimizer.step()
        del s1, s2, loss
        torch.cuda.synchronize()
        allocated.append(torch.cuda.memory_allocated())
    return losses, allocated, host(fc1.weight).copy(), host(fc2.weight).copy()


def test_training_loop_over_many_adam_steps(monkeypatch):
    steps = 60
    default = train_golden_network(steps, monkeypatch, {})
    plain = train_golden_network(steps, monkeypatch, {"PAIR_SPIKE_PSP": False, "PSP_RECURSION": False, "DENSE_EVENTS": False})
    for losses, allocated, w1, w2 in (default, plain):
        assert all(np.isfinite(losses)) and np.isfinite(w1).all() and np.isfinite(w2).all()
        # the loss comes down: the mean of the last ten steps is well below the mean of the first ten
        assert np.mean(losses[-10:]) < 0.8 * np.mean(losses[:10]), losses
        # nothing accumulates from step to step (pairing notes, kernel stamps, density readings)
        assert len(set(allocated[5:])) == 1, allocated
    # fused and recursive paths against the separate Functions over the tap sums: the same trajectory while
    # rounding differences have not yet moved a spike
    for a, b in zip(default[0][:10], plain[0][:10]):
        assert a == pytest.approx(b, rel=1e-4)


def test_pairing_notes_do_not_keep_tensors_alive_and_outputs_can_be_saved():
    """Layer outputs that require grad carry no Python state: torch.save works on them, and a note goes when its
    tensor does."""
    layer = snn.layer(neuron(), {"Ts": 1.0, "tSample": 300}).to(DEV)
    fc = layer.dense(20, 12, weightScale=60).to(DEV)
    x = (torch.rand((2, 20, 1, 1, 300), device=DEV) < 0.05).float()
    a = layer.psp(fc(x))
    s = layer.spike(fc(layer.psp(x)))
    assert a.requires_grad and s.requires_grad and not a.__dict__ and not s.__dict__
    for t in (a, s):
        buffer = io.BytesIO()
        torch.save(t, buffer)
        buffer.seek(0)
        assert torch.equal(torch.load(buffer, weights_only=True), t.detach())
    assert len(slayer_module._pspNotes) >= 1 and len(slayer_module._spikeNotes) >= 1
    before = (len(slayer_module._pspNotes), len(slayer_module._spikeNotes))
    del a, s, t
    assert (len(slayer_module._pspNotes), len(slayer_module._spikeNotes)) == (before[0] - 1, before[1] - 1)


def test_pairing_with_a_second_consumer_and_a_hook_gives_the_same_parameter_gradients(monkeypatch):
    """A hidden spike tensor with a second consumer and a gradient hook, a PSP signal with ``retain_grad``: the
    parameters' gradients are those of the separate Functions, the hook sees the whole gradient of the spikes (a
    watched tensor is not paired), and a potential changed in place after ``spike`` raises as in the reference."""
    layer = snn.layer(neuron(), {"Ts": 1.0, "tSample": 200}).to(DEV)
    torch.manual_seed(11)
    fc1, fc2 = layer.dense(30, 24, weightScale=70).to(DEV), layer.dense(24, 5, weightScale=70).to(DEV)
    rng = np.random.default_rng(12)
    x = dev((rng.random((2, 30, 1, 1, 200)) < 0.06).astype(np.float32))
    g = dev(rng.standard_normal((2, 5, 1, 1, 200)).astype(np.float32))
    gs = dev(rng.standard_normal((2, 24, 1, 1, 200)).astype(np.float32))

    def run(pair, watch):
        monkeypatch.setattr(slayer_module, "PAIR_SPIKE_PSP", pair)
        seen = {}
        for m in (fc1, fc2):
            m.weight.grad = None
        a1 = layer.psp(fc1(x))
        if watch:
            a1.retain_grad()
        s1 = layer.spike(a1)
        if watch:
            s1.register_hook(lambda grad: seen.__setitem__("s1", grad.clone()))
        a2 = layer.psp(s1)
        s2 = layer.spike(fc2(a2))
        ((layer.psp(s2) * g).sum() + (s1 * gs).sum()).backward()
        return fc1.weight.grad.clone(), fc2.weight.grad.clone(), seen.get("s1"), a1.grad if watch else None, \
            type(s1.grad_fn).__name__, type(a2.grad_fn).__name__

    apart, paired = run(False, False), run(True, False)
    assert float(apart[0].abs().sum()) > 0 and float(apart[1].abs().sum()) > 0
    assert paired[4] == "_spikeOfPspFunctionBackward" and apart[4] == "_spikeFunctionBackward"
    assert torch.equal(apart[1], paired[1]) and rel_err(host(paired[0]), host(apart[0])) <= 1e-5
    watched_apart, watched = run(False, True), run(True, True)
    assert watched[4] == "_spikeFunctionBackward" and watched[5] == "_pspFunctionBackward"     # not paired
    for a, b in zip(watched_apart[:4], watched[:4]):
        assert a is not None and torch.equal(a, b)
    assert torch.equal(watched[0], apart[0]) and torch.equal(watched[1], apart[1])

    monkeypatch.setattr(slayer_module, "PAIR_SPIKE_PSP", True)
    u = (fc1(layer.psp(x)) * 1.0)
    s = layer.spike(u)
    u.add_(1.0)                                        # the saved potential is no longer what the spikes came from
    a = layer.psp(s)
    assert type(a.grad_fn).__name__ == "_pspFunctionBackward"
    with pytest.raises(RuntimeError, match="modified by an inplace operation"):
        a.sum().backward()


def test_dense_layer_density_follows_the_input_without_waiting(monkeypatch):
    """DENSE_EVENTS = "auto": a layer whose first batches are silent and whose later batches are dense leaves the
    event kernels within a few calls, and comes back; a new input shape is measured at once; results are those of
    the library product either way."""
    monkeypatch.setattr(slayer_module, "DENSE_EVENTS", "auto")
    monkeypatch.setattr(slayer_module, "DENSE_EVENTS_MIN_CHANNELS", 64)
    layer = snn.layer(neuron(), {"Ts": 1.0, "tSample": 128}).to(DEV)
    torch.manual_seed(3)
    fc = layer.dense(256, 32).to(DEV)
    sparse = (torch.rand((2, 256, 1, 1, 128), device=DEV) < 0.01).float()
    dense = (torch.rand((2, 256, 1, 1, 128), device=DEV) < 0.5).float()

    def check(x):
        want = torch.nn.functional.conv3d(x, fc.weight)
        assert rel_err(host(fc(x)), host(want)) < 1e-5
        torch.cuda.synchronize()

    check(sparse)
    assert fc._eventDensity == pytest.approx(float(sparse.mean()), rel=1e-6) and fc._inputIsSparse(sparse.reshape(2, 256, 128)) == (True, True)
    for _ in range(2 * slayer_module.DENSE_EVENTS_CHECK_EVERY + 2):
        check(dense)
    assert fc._eventDensity == pytest.approx(float(dense.mean()), rel=1e-6)
    for _ in range(2 * slayer_module.DENSE_EVENTS_CHECK_EVERY + 2):
        check(sparse)
    assert fc._eventDensity == pytest.approx(float(sparse.mean()), rel=1e-6)
    other = (torch.rand((3, 256, 1, 1, 96), device=DEV) < 0.4).float()
    check(other)                                        # a new shape: measured in that very call
    assert fc._eventDensity == pytest.approx(float(other.mean()), rel=1e-6)


# ------------------------------------------------------------------------------ HIP graph replay
@pytest.mark.parametrize("N,T", [(3, 100), (4, 512)], ids=["library dense products", "dense layers on the matrix-core kernels"])
def test_training_step_replayed_by_capturedStep(N, T):
    """A whole training step - psp, spike, delay, dense, loss, backward - recorded by ``utils.capturedStep``.
    Every replay, with eager work and synchronisations in between, must reproduce the eager step bit for bit.  At
    (4, 512) the first dense layer runs synapse.denseRows and denseRowsGradWeight (workspaces from torch's allocator
    inside the capture)."""
    params = {"type": "SRMALPHA", "theta": 10, "tauSr": 4.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    sim = {"Ts": 1.0, "tSample": T}
    layer = snn.layer(params, sim).cuda()
    error = snn.loss({"neuron": params, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}).cuda()
    torch.manual_seed(2)
    fc1, fc2 = layer.dense(40, 32, weightScale=30).cuda(), layer.dense(32, 6, weightScale=30).cuda()
    delay = layer.delay(32).cuda()
    x = (torch.rand((N, 40, 1, 1, T)) < 0.1).float().cuda()
    x2 = (torch.rand((N, 40, 1, 1, T)) < 0.1).float().cuda()
    target = (torch.rand((N, 6, 1, 1, T)) < 0.05).float().cuda()
    from slayerpytorch_amd import synapse
    assert synapse.denseRowsPays(N, 40, 32, T) == (N * T >= 2048)
    batch = x.clone()
    leaves = [fc1.weight, fc2.weight, delay.delay]
    for p in leaves:
        p.grad = torch.zeros_like(p)

    def step():
        for p in leaves:
            p.grad.zero_()
        s1 = layer.spikeDelayed(layer.psp(fc1(batch)), delay)
        s2 = layer.spike(layer.psp(fc2(s1)))
        loss = error.spikeTime(s2, target)
        loss.backward()
        return loss

    def eager(data):
        batch.copy_(data)
        loss = step()
        torch.cuda.synchronize()
        return [loss.detach().clone()] + [p.grad.clone() for p in leaves]

    refs = {id(x): eager(x), id(x2): eager(x2)}
    assert all(float(r.abs().sum()) > 0 for r in refs[id(x)]) and not torch.equal(refs[id(x)][0], refs[id(x2)][0])
    replayed = capturedStep(step)
    for data in (x, x2, x, x2):
        batch.copy_(data)
        static_loss = replayed()
        torch.cuda.synchronize()
        got = [static_loss.detach()] + [p.grad for p in leaves]
        for a, b in zip(got, refs[id(data)]):
            assert torch.equal(a, b)
        again = eager(data)                   # the program's own eager work between replays
        for a, b in zip(again, refs[id(data)]):
            assert torch.equal(a, b)
    replayed.reset()
    batch.copy_(x)
    assert torch.equal(replayed().detach(), refs[id(x)][0])


# ----------------------------------------------------------- full batch sizes against the oracle chain
# How these tests deal with the threshold.  GPU and oracle round the potential differently (recursion against tap
# sums, fp32 against double accumulation in the synapse), so a spike may flip where the potential sits within that
# rounding of theta, and one flip moves the spikes that follow it in its row.  Every oracle stage therefore gets
# the input its GPU counterpart had (the oracle's layer 2 filters the GPU's layer-1 spikes, the oracle's backward
# pass uses the potentials the GPU saved), the flips of each layer are counted and bounded, and each row's first
# flip must sit at a potential within FLIP_BAND of the threshold - anything else is a wrong spike, not rounding.
FLIP_RATE_MAX = 1e-5     # per layer, on identical layer inputs (the first layers measure 5e-7 or less)
FLIP_BAND = 2e-4         # |u - theta| / theta at a row's first flip
POTENTIAL_TOL = 2e-6     # max |u_gpu - u_oracle| / max |u_oracle| before the spike function


def check_spikes(s_gpu, u_gpu_before, o_s, o_u_before, o_u_after, theta):
    """Potentials before the spike function agree to rounding; spikes are identical except for rows whose first
    difference sits at the threshold; returns the flip rate."""
    assert rel_err(u_gpu_before, o_u_before) <= POTENTIAL_TOL
    T = o_s.shape[-1]
    diff = (s_gpu != o_s).reshape(-1, T)
    rows = np.nonzero(diff.any(axis=1))[0]
    first = diff[rows].argmax(axis=1)
    at_flip = o_u_after.reshape(-1, T)[rows, first]      # (what the oracle compared with theta at that sample)
    assert np.all(np.abs(at_flip - theta) <= FLIP_BAND * theta), np.abs(at_flip - theta).max()
    rate = float(diff.sum()) / diff.size
    assert rate <= FLIP_RATE_MAX, rate
    return rate


def oracle_spike_loss_grad(s_out, target, srm, Ts):
    """Gradient of 1/2 * sum(psp(s - target)^2) * Ts with respect to s (src/spikeLoss.py:56-58), and the loss."""
    e = O.conv(s_out - target, srm, Ts)
    loss = 0.5 * float(np.sum(e.astype(np.float64) ** 2)) * Ts
    return O.corr(e * np.float32(Ts), srm, Ts), loss


def test_nmnist_mlp_step_at_full_batch_matches_the_oracle_chain():
    """One training step of the NMNIST-shaped MLP (example/02_NMNIST_MLP/nmnistMLP.py:59-60: spike(psp(fc(.)))
    twice, spike-time loss) on Bernoulli(0.015) input (12, 2, 34, 34, 350): potentials and spikes of both layers,
    the loss and both weight gradients (norm-wise within 1e-4) against the oracle chain."""
    Ts, T = 1.0, 350
    nd = neuron()
    sim = {"Ts": Ts, "tSample": T}
    layer = snn.layer(nd, sim).to(DEV)
    error = snn.loss({"neuron": nd, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}).to(DEV)
    rng = np.random.default_rng(20)
    x = (rng.random((12, 2, 34, 34, T)) < 0.015).astype(np.float32)
    w1 = (rng.standard_normal((512, 2, 34, 34)) * 0.35).astype(np.float32)
    w2 = (rng.standard_normal((10, 512, 1, 1)) * 1.2).astype(np.float32)
    target = np.zeros((12, 10, 1, 1, T), dtype=np.float32)
    target[np.arange(12), rng.integers(0, 10, 12), 0, 0, :] = (rng.random((12, T)) < 0.1)
    fc1, fc2 = layer.dense((34, 34, 2), 512).to(DEV), layer.dense(512, 10).to(DEV)
    fc1.weight = torch.nn.Parameter(dev(w1).reshape(512, 2, 34, 34, 1))
    fc2.weight = torch.nn.Parameter(dev(w2).reshape(10, 512, 1, 1, 1))
    u1 = layer.psp(fc1(dev(x)))
    u1_before = host(u1).copy()
    s1 = layer.spike(u1)                       # (u1 now holds the potential after the refractory responses)
    u2 = layer.psp(fc2(s1))
    u2_before = host(u2).copy()
    s2 = layer.spike(u2)
    loss = error.spikeTime(s2, dev(target))
    loss.backward()

    srm, ref = host(layer.srmKernel), host(layer.refKernel)
    theta, tau, scale = nd["theta"], nd["tauRho"] * nd["theta"], nd["scaleRho"]
    O.set_threads(O.max_threads())
    try:
        o_u1 = O.conv(O.synapse_conv(x, w1), srm, Ts)
        o_s1, o_u1_after = O.get_spikes(o_u1, ref, theta, Ts)
        check_spikes(host(s1), u1_before, o_s1, o_u1, o_u1_after, theta)
        o_u2 = O.conv(O.synapse_conv(host(s1), w2), srm, Ts)
        o_s2, o_u2_after = O.get_spikes(o_u2, ref, theta, Ts)
        check_spikes(host(s2), u2_before, o_s2, o_u2, o_u2_after, theta)
        assert 0.01 < o_s1.mean() < 0.3 and 0.01 < o_s2.mean() < 0.5, (o_s1.mean(), o_s2.mean())     # both layers are active
        g_s2, o_loss = oracle_spike_loss_grad(host(s2), target, srm, Ts)
        g_a2 = O.corr(O.spike_bwd(g_s2, host(u2), theta, tau, scale), srm, Ts)
        g_w2 = O.synapse_conv_grad_weight(g_a2, host(s1), w2.shape)
        g_s1 = O.synapse_conv_grad_input(g_a2, w2, s1.shape)
        g_a1 = O.corr(O.spike_bwd(g_s1, host(u1), theta, tau, scale), srm, Ts)
        g_w1 = O.synapse_conv_grad_weight(g_a1, x, w1.shape)
    finally:
        O.set_threads(1)
    assert float(loss.detach()) == pytest.approx(o_loss, rel=1e-4)
    assert rel_err(host(fc2.weight.grad).reshape(g_w2.shape), g_w2) < 1e-4
    assert rel_err(host(fc1.weight.grad).reshape(g_w1.shape), g_w1) < 1e-4


def test_nmnist_cnn_first_layers_at_full_batch_match_the_oracle_chain():
    """The first two layers of the NMNIST-shaped CNN (example/03_NMNIST_CNN/nmnistCNN.py:55-58: spike(conv1(psp(x))),
    spike(pool1(psp(.)))) on Bernoulli(0.02) input (12, 2, 34, 34, 300), and the PSP of the pooled spikes against a
    random cotangent: potentials and spikes of both layers, the convolution's weight gradient and the input
    gradient (norm-wise within 1e-4) against the oracle chain."""
    Ts, T = 1.0, 300
    nd = neuron()
    layer = snn.layer(nd, {"Ts": Ts, "tSample": T}).to(DEV)
    rng = np.random.default_rng(21)
    x = (rng.random((12, 2, 34, 34, T)) < 0.02).astype(np.float32)
    w1 = (rng.standard_normal((16, 2, 5, 5)) * 1.5).astype(np.float32)
    g = rng.standard_normal((12, 16, 17, 17, T)).astype(np.float32)
    conv1, pool1 = layer.conv(2, 16, 5, padding=2).to(DEV), layer.pool(2).to(DEV)
    conv1.weight = torch.nn.Parameter(dev(w1).reshape(16, 2, 5, 5, 1))
    xin = dev(x).requires_grad_(True)
    u1 = conv1(layer.psp(xin))
    u1_before = host(u1).copy()
    s1 = layer.spike(u1)
    u2 = pool1(layer.psp(s1))
    u2_before = host(u2).copy()
    s2 = layer.spike(u2)
    (layer.psp(s2) * dev(g)).sum().backward()

    srm, ref = host(layer.srmKernel), host(layer.refKernel)
    theta, tau, scale = nd["theta"], nd["tauRho"] * nd["theta"], nd["scaleRho"]
    wp = np.full((1, 1, 2, 2), np.float32(1.1 * theta), dtype=np.float32)
    O.set_threads(O.max_threads())
    try:
        p0 = O.conv(x, srm, Ts)
        o_u1 = O.synapse_conv(p0, w1, 1, 2)
        o_s1, o_u1_after = O.get_spikes(o_u1, ref, theta, Ts)
        check_spikes(host(s1), u1_before, o_s1, o_u1, o_u1_after, theta)
        p1 = O.conv(host(s1), srm, Ts).reshape(12, 1, 16 * 34, 34, T)
        o_u2 = O.synapse_conv(p1, wp, 2, 0).reshape(12, 16, 17, 17, T)
        o_s2, o_u2_after = O.get_spikes(o_u2, ref, theta, Ts)
        check_spikes(host(s2), u2_before, o_s2, o_u2, o_u2_after, theta)
        assert 0.01 < o_s1.mean() < 0.3 and 0.01 < o_s2.mean() < 0.6, (o_s1.mean(), o_s2.mean())   # (a pooled layer fires on every input spike)
        g_u2 = O.spike_bwd(O.corr(g, srm, Ts), host(u2), theta, tau, scale)
        g_p1 = O.synapse_conv_grad_input(g_u2.reshape(12, 1, 16 * 17, 17, T), wp, p1.shape, 2, 0).reshape(o_s1.shape)
        g_u1 = O.spike_bwd(O.corr(g_p1, srm, Ts), host(u1), theta, tau, scale)
        g_w1 = O.synapse_conv_grad_weight(g_u1, p0, w1.shape, 1, 2)
        g_x = O.corr(O.synapse_conv_grad_input(g_u1, w1, p0.shape, 1, 2), srm, Ts)
    finally:
        O.set_threads(1)
    assert rel_err(host(conv1.weight.grad).reshape(g_w1.shape), g_w1) < 1e-4
    assert rel_err(host(xin.grad), g_x) < 1e-4

"""Pins the CPU oracle (oracle/slayer_oracle.c) before anything is compared against it:
golden vectors held by the reference's own tests, library routines the ops reduce to,
closed forms, invariants and brute force on small inputs.  Runs without a GPU.
"""
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O
from slayerpytorch_amd.slayer import alphaKernel
from slayerpytorch_amd.slayerLoihi import loihiPspKernel, loihiRefKernel

from _util import golden, raster_from_aer, raster_from_events, rel_err

rng = np.random.default_rng(1234)


# ------------------------------------------------------------------------------------------
# kernel generators (host code, pinned by reference-held tables and the documented lengths)
# ------------------------------------------------------------------------------------------
def test_alpha_kernels_match_reference_tables():
    snn = golden("snn_250_25_1.npz")
    tv = golden("torch_validate.npz")
    srm = np.array(alphaKernel(1.0, 0.1, 50))
    ref = np.array(alphaKernel(1.0, 0.1, 50, mult=-20))
    assert len(srm) == 77 and len(ref) == 110
    # tables are printed with 4 decimals
    assert np.abs(snn["h_sr"][:, 1] - srm).max() < 6e-5
    assert np.abs(snn["h_ref"][:, 1] - ref).max() < 6e-5
    assert np.abs(snn["h_sr"][:, 0] - 0.1 * np.arange(77)).max() < 1e-6
    # 5 significant digits
    assert np.abs(tv["refractory_kernel"] - ref).max() < 6e-4


@pytest.mark.parametrize("tau,Ts,mult,eps,length", [
    (10.0, 1.0, 1, 0.01, 77), (1.0, 1.0, 1, 0.01, 8), (1.0, 1.0, -20, 0.01, 11),
    (1.0, 0.1, 1, 0.01, 77), (1.0, 0.1, -20, 0.01, 110), (1.0, 0.1, -20, 0.0001, 160)])
def test_alpha_kernel_lengths(tau, Ts, mult, eps, length):
    k = alphaKernel(tau, Ts, 300, mult=mult, EPSILON=eps)
    assert len(k) == length
    assert k[0] == 0
    peak = int(round(tau / Ts))
    assert k[peak] == pytest.approx(mult)           # t/tau * exp(1 - t/tau) peaks at t = tau with value 1


def test_alpha_kernel_is_cut_by_tSample():
    assert len(alphaKernel(10.0, 1.0, 20)) == 20


def test_loihi_kernels():
    psp = loihiPspKernel(1024, 128, 0)
    assert psp[:5] == [64.0, 110.0, 142.5, 165.0, 179.5]
    assert len(psp) == 110 and max(psp) == 195.0 and psp[-1] == 0.0
    # twice the PSP kernel is the voltage a Loihi chip recorded for one weight-2 input spike
    chip = golden("loihi_chip.npz")["impulseVoltage"]
    assert np.array_equal((2 * np.array(psp)).astype(int)[: len(chip) - 1], chip[1:])
    ref = loihiRefKernel(5120, 128, 3)
    assert ref[0] == 0 and ref[1] == ref[2] == -5120000 and ref[3] == -10240 and ref[4] == -2 * ((5120 * 3968) >> 12)
    assert ref[-1] == 0


# ------------------------------------------------------------------------------------------
# conv / corr
# ------------------------------------------------------------------------------------------
@pytest.mark.parametrize("T,Fl", [(50, 7), (300, 77), (8, 20), (1, 1), (33, 2)])
@pytest.mark.parametrize("fused", [True, False])
def test_conv_is_numpy_convolve(T, Fl, fused):
    x = rng.standard_normal((5, T)).astype(np.float32)
    f = rng.standard_normal(Fl).astype(np.float32)
    Ts = 0.5
    want = np.stack([np.convolve(r.astype(np.float64), f.astype(np.float64))[:T] for r in x]) * Ts
    got = O.conv(x, f, Ts, fused=fused)
    assert rel_err(got, want) < 1e-6


@pytest.mark.parametrize("T,Fl", [(50, 7), (300, 77), (8, 20), (1, 1)])
def test_corr_is_numpy_correlate(T, Fl):
    x = rng.standard_normal((4, T)).astype(np.float32)
    f = rng.standard_normal(Fl).astype(np.float32)
    Ts = 2.0
    want = np.stack([np.correlate(np.concatenate([r, np.zeros(Fl - 1)]).astype(np.float64),
                                  f.astype(np.float64), mode="valid") for r in x]) * Ts
    assert rel_err(O.corr(x, f, Ts), want) < 1e-6


def test_conv_is_left_padded_conv3d_with_flipped_filter():
    # the identity the reference asserts between slayer.psp and pspLayer
    x = torch.from_numpy(rng.standard_normal((2, 3, 4, 5, 60)).astype(np.float32))
    f = torch.from_numpy(np.array(alphaKernel(10.0, 1.0, 60), dtype=np.float32))
    Ts = 1.0
    padded = F.pad(x.reshape(2, 1, 1, -1, 60), (f.numel() - 1, 0))
    want = (F.conv3d(padded, torch.flip(f, [0]).reshape(1, 1, 1, 1, -1)) * Ts).reshape(x.shape)
    got = O.conv(x.numpy(), f.numpy(), Ts)
    assert rel_err(got, want.numpy()) < 1e-6


def test_conv_corr_adjoint_linearity_causality_impulse():
    T, Fl, Ts = 40, 9, 0.25
    f = rng.standard_normal(Fl).astype(np.float32)
    x = rng.standard_normal((3, T)).astype(np.float32)
    y = rng.standard_normal((3, T)).astype(np.float32)
    lhs = np.sum(O.conv(x, f, Ts).astype(np.float64) * y)
    rhs = np.sum(x * O.corr(y, f, Ts).astype(np.float64))
    assert abs(lhs - rhs) < 1e-4 * max(1.0, abs(lhs))
    a, b = 1.5, -0.75
    assert rel_err(O.conv(a * x + b * y, f, Ts), a * O.conv(x, f, Ts) + b * O.conv(y, f, Ts)) < 1e-6
    imp = np.zeros((1, T), np.float32)
    imp[0, 5] = 4.0
    out = O.conv(imp, f, Ts)[0]
    assert np.all(out[:5] == 0)                                   # causal
    np.testing.assert_allclose(out[5:5 + Fl], 4.0 * f * Ts, rtol=1e-6)
    out = O.corr(imp, f, Ts)[0]
    assert np.all(out[6:] == 0)                                   # anti-causal
    np.testing.assert_allclose(out[5::-1][: min(6, Fl)], 4.0 * f[:6] * Ts, rtol=1e-6)


def test_conv_golden_vectors():
    tv = golden("torch_validate.npz")
    srm = np.array(alphaKernel(1.0, 0.1, 50), dtype=np.float32)
    s1 = raster_from_events(tv["s1_shape"], tv["s1_events"], tv["s1_values"])
    # files carry 5 significant digits
    assert np.abs(O.conv(s1, srm, 0.1) - tv["a1"]).max() < 1e-4
    assert np.abs(O.conv(tv["s3"], srm, 0.1) - tv["a3"]).max() < 1e-4
    assert np.abs(O.conv(tv["des_s"], srm, 0.1) - tv["des_a"]).max() < 1e-4
    nm = golden("nmnist_response.npz")
    b = raster_from_events(nm["binned_shape"], nm["binned_events"], nm["binned_values"])
    assert np.abs(O.conv(b, np.array(alphaKernel(1.0, 1.0, 350), np.float32), 1.0) - nm["response"]).max() < 1e-4
    b2 = raster_from_events(nm["binned_ts2_shape"], nm["binned_ts2_events"], nm["binned_ts2_values"])
    assert np.abs(O.conv(b2, np.array(alphaKernel(1.0, 2.0, 350), np.float32), 2.0) - nm["response_ts2"]).max() < 1e-4


# ------------------------------------------------------------------------------------------
# spike
# ------------------------------------------------------------------------------------------
def brute_spikes(u, nu, theta, Ts):
    """Per-neuron loop in the spirit of the numpy check of the reference's test_slayer002."""
    u = u.astype(np.float32).copy()
    s = np.zeros_like(u)
    T = u.shape[-1]
    flat_u, flat_s = u.reshape(-1, T), s.reshape(-1, T)
    for r in range(flat_u.shape[0]):
        for t in range(T):
            if flat_u[r, t] >= np.float32(theta):
                flat_s[r, t] = np.float32(1.0) / np.float32(Ts)
                n = min(len(nu), T - t)
                flat_u[r, t:t + n] = flat_u[r, t:t + n] + nu[:n]
    return s, u


@pytest.mark.parametrize("T,nuSize", [(64, 11), (37, 1), (20, 40), (5, 0), (100, 33)])
def test_spikes_match_brute_force_bitwise(T, nuSize):
    u = (rng.standard_normal((2, 3, 2, 2, T)) * 6).astype(np.float32)
    nu = (-rng.random(nuSize) * 15).astype(np.float32)
    s, ua = O.get_spikes(u, nu, 10.0, 0.5)
    sb, ub = brute_spikes(u, nu, 10.0, 0.5)
    assert np.array_equal(s, sb) and np.array_equal(ua.view(np.uint32), ub.view(np.uint32))
    assert set(np.unique(s)) <= {0.0, 2.0}


def test_spike_special_cases():
    u = (rng.standard_normal((1, 1, 1, 4, 30)) * 6).astype(np.float32)
    nu = np.array([0, -20, -15, -3], np.float32)
    s, ua = O.get_spikes(u, nu, np.inf, 1.0)
    assert not s.any() and np.array_equal(ua, u)
    one = np.zeros((1, 1, 1, 1, 12), np.float32)
    one[..., 4] = 10.0                                   # exactly at threshold fires (>=)
    s, ua = O.get_spikes(one, nu, 10.0, 1.0)
    assert s[..., 4] == 1.0 and s.sum() == 1.0
    want = one.copy()
    want[..., 4:8] += nu
    assert np.array_equal(ua, want)
    one[..., 4] = np.nextafter(np.float32(10.0), np.float32(0))
    assert not O.get_spikes(one, nu, 10.0, 1.0)[0].any()
    # clipping at the end of the row
    end = np.zeros((1, 1, 1, 1, 6), np.float32)
    end[..., 4] = 11.0
    s, ua = O.get_spikes(end, nu, 10.0, 1.0)
    assert np.array_equal(ua[0, 0, 0, 0], np.array([0, 0, 0, 0, 11, -20], np.float32))


def test_spike_golden_triples():
    snn = golden("snn_250_25_1.npz")
    ref = np.array(alphaKernel(1.0, 0.1, 50, mult=-20, EPSILON=0.0001), dtype=np.float32)   # fullRefKernel
    for key, nspikes in (("spikeFuncHid", 20), ("spikeFuncHid04", 13), ("spikeFuncOut", 3)):
        d = snn[key]                       # columns: u before refractory, u after, spike
        s, ua = O.get_spikes(d[None, None, None, None, :, 0], ref, 10.0, 0.1)
        assert np.array_equal(s.reshape(-1), d[:, 2]), key
        assert (d[:, 2] > 0).sum() == nspikes
        assert np.abs(ua.reshape(-1) - d[:, 1]).max() < 1e-3, key        # 6 significant digits in the file


def test_spike_chain_golden_250_25_1():
    """spikeIn -> psp -> dense -> spike == spikeHid; -> dense -> psp -> spike == spikeOut
    (the data the reference's test_slayer002 loads)."""
    snn = golden("snn_250_25_1.npz")
    Ts, Ns = 0.1, 500
    srm = np.array(alphaKernel(1.0, Ts, 50), dtype=np.float32)
    ref = np.array(alphaKernel(1.0, Ts, 50, mult=-20, EPSILON=0.0001), dtype=np.float32)
    x = raster_from_aer(snn["spikeIn"], 250, Ns, Ts, 1 / Ts)
    uHid = (snn["w1learned"].astype(np.float64) @ O.conv(x, srm, Ts).astype(np.float64)).astype(np.float32)
    sHid, _ = O.get_spikes(uHid.reshape(1, 25, 1, 1, Ns), ref, 10.0, Ts)
    want = raster_from_aer(snn["spikeHid"], 25, Ns, Ts, 1 / Ts)
    assert len(snn["spikeHid"]) == 289
    assert np.array_equal(sHid.reshape(25, Ns), want)
    uOut = O.conv((snn["w2learned"].astype(np.float64) @ sHid.reshape(25, Ns)).astype(np.float32), srm, Ts)
    sOut, _ = O.get_spikes(uOut.reshape(1, 1, 1, 1, Ns), ref, 10.0, Ts)
    assert np.array_equal(np.nonzero(sOut.reshape(-1))[0], np.array([203, 355, 447]))


def test_spike_chain_golden_torch_validate():
    tv = golden("torch_validate.npz")
    Ts = 0.1
    ref = np.array(alphaKernel(1.0, Ts, 50, mult=-20, EPSILON=0.0001), dtype=np.float32)
    u2 = (tv["W12"].astype(np.float64) @ tv["a1"].astype(np.float64)).astype(np.float32)
    s2, u2r = O.get_spikes(u2.reshape(1, 25, 1, 1, -1), ref, 10.0, Ts)
    assert np.array_equal(s2.reshape(25, -1), tv["s2"]) and (tv["s2"] > 0).sum() == 266
    assert np.abs(u2r.reshape(25, -1) - tv["u2"]).max() < 2e-2      # a1 itself carries 5 digits


def test_output_layer_and_gradients_golden_torch_validate():
    """The rest of the legacy traces of the 250-25-1 network (Ts = 0.1): the output neuron's potential and spikes
    (u3, s3: 11 spikes) from the hidden spikes, its filtered spikes a3, the error signal e3 against the desired
    response, and both weight gradients - a second joint pin of conv, spike, spike pdf and corr:
    delta3 = pdf(u3) * corr(e3), Wgrad2 = Ts * delta3 a2^T, delta2 = pdf(u2) * corr(W23^T delta3),
    Wgrad1 = Ts * delta2 a1^T.  Tolerances are those of 5-digit CSV files."""
    tv = golden("torch_validate.npz")
    Ts, theta, tau = 0.1, 10.0, 4.3429
    srm = np.array(alphaKernel(1.0, Ts, 50), dtype=np.float32)
    ref = tv["refractory_kernel"]
    a2 = O.conv(tv["s2"].reshape(1, 25, 1, 1, -1), srm, Ts).reshape(25, -1)
    pre3 = (tv["W23"].astype(np.float64) @ a2.astype(np.float64)).astype(np.float32)
    s3, u3 = O.get_spikes(pre3.reshape(1, 1, 1, 1, -1), ref, theta, Ts)
    assert np.array_equal(s3.reshape(1, -1), tv["s3"]) and (tv["s3"] > 0).sum() == 11
    assert np.abs(u3.reshape(1, -1) - tv["u3"]).max() < 2e-2
    a3 = O.conv(s3, srm, Ts).reshape(1, -1)
    assert np.abs(a3 - tv["a3"]).max() < 1e-4
    assert np.abs((a3 - tv["des_a"]) - tv["e3"]).max() < 2e-4
    d3 = O.spike_bwd(O.corr(tv["e3"].reshape(1, 1, 1, 1, -1), srm, Ts), tv["u3"].reshape(1, 1, 1, 1, -1), theta, tau, 1.0)
    d3 = d3.reshape(1, -1)
    g2 = (d3.astype(np.float64) @ a2.astype(np.float64).T) * Ts
    assert rel_err(g2, tv["Wgrad2"]) < 1e-4
    e2 = (tv["W23"].astype(np.float64).T @ d3.astype(np.float64)).astype(np.float32)
    d2 = O.spike_bwd(O.corr(e2.reshape(1, 25, 1, 1, -1), srm, Ts), tv["u2"].reshape(1, 25, 1, 1, -1), theta, tau, 1.0)
    g1 = (d2.reshape(25, -1).astype(np.float64) @ tv["a1"].astype(np.float64).T) * Ts
    assert rel_err(g1, tv["Wgrad1"]) < 2e-4


# ------------------------------------------------------------------------------------------
# spike pdf backward
# ------------------------------------------------------------------------------------------
def test_spike_bwd_closed_form_and_golden():
    u = (rng.standard_normal(1000) * 8).astype(np.float32)
    g = rng.standard_normal(1000).astype(np.float32)
    theta, tau, scale = 10.0, 4.3429, 1.0
    want = g.astype(np.float64) * scale / tau * np.exp(-np.abs(u.astype(np.float64) - theta) / tau)
    assert rel_err(O.spike_bwd(g, u, theta, tau, scale), want) < 1e-6
    tv = golden("torch_validate.npz")
    rho = O.spike_bwd(np.ones_like(tv["u3"]), tv["u3"], theta, tau, scale)
    assert np.abs(rho - tv["rho3"]).max() < 5e-5 and tv["rho3"].max() == pytest.approx(0.22861)


# ------------------------------------------------------------------------------------------
# shift
# ------------------------------------------------------------------------------------------
def slice_shift(row, k):
    out = np.zeros_like(row)
    T = len(row)
    if k == 0:
        out[:] = row
    elif 0 < k < T:
        out[k:] = row[:-k]
    elif -T < k < 0:
        out[:k] = row[-k:]
    return out


def test_shift_per_neuron_exact():
    N, C, H, W, T, Ts = 3, 4, 3, 2, 50, 0.1
    x = rng.standard_normal((N, C, H, W, T)).astype(np.float32)
    d = (rng.random((C, H, W)) * 2 - 1).astype(np.float32)
    d.reshape(-1)[:4] = [0.0, -0.25, 0.3, 7.0]            # zero, truncation toward zero, boundary, beyond the row
    out = O.shift(x, d, Ts)
    for n in range(N):
        for c in range(C):
            for h in range(H):
                for w in range(W):
                    k = int(np.float32(d[c, h, w]) / np.float32(Ts))
                    assert np.array_equal(out[n, c, h, w], slice_shift(x[n, c, h, w], k))
    assert int(np.float32(-0.25) / np.float32(0.1)) == -2


def test_shift_scalar_and_roundtrip():
    x = rng.standard_normal((2, 3, 1, 1, 40)).astype(np.float32)
    out = O.shift(x, 4, 1.0)
    assert np.array_equal(out[..., 4:], x[..., :-4]) and not out[..., :4].any()
    back = O.shift(out, -4, 1.0)
    assert np.array_equal(back[..., :-4], x[..., :-4]) and not back[..., -4:].any()
    same = O.shift(x, np.full((3, 1, 1), 4, np.float32), 1.0)
    assert np.array_equal(same, out)
    with pytest.raises(ValueError):
        O.shift(x, np.zeros(5, np.float32), 1.0)


# ------------------------------------------------------------------------------------------
# delay gradient
# ------------------------------------------------------------------------------------------
def test_delay_grad_formula():
    N, C, T, Ts = 4, 6, 80, 0.1
    y = rng.standard_normal((N, C, 1, 1, T))
    g = rng.standard_normal((N, C, 1, 1, T))
    yf, gf = y.astype(np.float32), g.astype(np.float32)
    # -sum(e * d/dt y) * Ts with the backward difference d/dt y[t] = (y[t] - y[t-1]) / Ts
    dy = (yf.astype(np.float64) - np.concatenate([np.zeros_like(y[..., :1]), yf[..., :-1].astype(np.float64)], -1)) / Ts
    want = -(gf.astype(np.float64) * dy).sum(axis=(0, -1)) * Ts
    got = O.delay_grad(yf, gf, Ts)
    assert got.shape == (C, 1, 1)
    assert rel_err(got, want) < 1e-5


# ------------------------------------------------------------------------------------------
# Loihi neuron
# ------------------------------------------------------------------------------------------
def numpy_loihi(w, wgtExp, theta, iDecay, vDecay, refDelay):
    """Vectorised integer model with an explicit spike look-back, after the numpy model that the
    reference's test_slayerLoihi002 checks the CUDA kernel against."""
    w = np.asarray(w)
    T = w.shape[-1]
    flat = w.reshape(-1, T)
    n = flat.shape[0]
    cur = np.zeros((n, T), np.int64)
    vol = np.zeros((n, T), np.int64)
    spk = np.zeros((n, T), np.int64)
    ref = np.zeros(n, np.int64)
    scale = 1 << (6 + wgtExp)
    M = 0xFFFFFFFF

    def wrap(x):                     # 32-bit two's complement, as the kernel's int variables
        return ((x + (1 << 31)) & M) - (1 << 31)

    for t in range(1, T):
        cs = np.where(cur[:, t - 1] >= 0, 1, -1)
        vs = np.where(vol[:, t - 1] >= 0, 1, -1)
        # the magnitude product is a 32-bit unsigned value (it wraps once |state| >= 2**20)
        cur[:, t] = wrap(cs * (((cs * cur[:, t - 1] * (4096 - iDecay)) & M) >> 12)
                         + scale * np.trunc(flat[:, t]).astype(np.int64))
        vol[:, t] = wrap(vs * (((vs * vol[:, t - 1] * (4096 - vDecay)) & M) >> 12) + cur[:, t])
        if t >= refDelay:
            ref -= spk[:, t - refDelay]
        spk[:, t] = (vol[:, t] > theta) & (ref == 0)
        vol[:, t] *= (1 - spk[:, t]) * (ref == 0)
        ref += spk[:, t]
    vout = (1 - spk) * vol + spk * vDecay
    return (spk.reshape(w.shape).astype(np.float32), vout.reshape(w.shape).astype(np.float32),
            cur.reshape(w.shape).astype(np.float32))


@pytest.mark.parametrize("refDelay", [1, 2, 5, 17])
def test_loihi_matches_numpy_model(refDelay):
    numSrc, numDst, T = 128, 64, 200
    weight = np.round((rng.random((numDst, numSrc)) - 0.5) * 10) * 2
    spikes = rng.random((numSrc, T)) > 0.8
    w = weight.dot(spikes).astype(np.float32)
    got = O.loihi_get_spikes(w, 0, 80 * 64, 1024, 128, refDelay)
    want = numpy_loihi(w, 0, 80 * 64, 1024, 128, refDelay)
    for a, b, name in zip(got, want, ("spike", "voltage", "current")):
        assert np.array_equal(a, b), name
    assert got[0].sum() > 0
    assert not got[0][:, 0].any() and not got[2][:, 0].any()        # t = 0 is forced to zero


def test_loihi_other_parameters_and_negative_truncation():
    w = (rng.standard_normal((3, 5, 90)) * 40).astype(np.float32)      # non-integers: truncation toward zero
    for wgtExp, theta, iDecay, vDecay, refDelay in [(1, 10 * 64, 2048, 256, 3), (0, 64, 0, 0, 1), (2, 5000, 4095, 4095, 2)]:
        got = O.loihi_get_spikes(w, wgtExp, theta, iDecay, vDecay, refDelay)
        want = numpy_loihi(w, wgtExp, theta, iDecay, vDecay, refDelay)
        for a, b in zip(got, want):
            assert np.array_equal(a, b)
    with pytest.raises(ValueError):
        O.loihi_get_spikes(w, 0, 64, 0, 0, 0)


def test_loihi_chip_recordings():
    """dense -> Loihi -> shift(1) -> dense -> Loihi -> shift(1) against spikes and voltages
    recorded from a Loihi chip (the data of the reference's test_slayerLoihi001)."""
    snn, chip = golden("snn_250_25_1.npz"), golden("loihi_chip.npz")
    Ts, Ns, theta = 0.1, 500, 80 * 64
    x = raster_from_aer(snn["spikeIn"], 250, Ns, Ts, 1 / Ts, offset=49)
    W1 = np.round(snn["w1learned"].astype(np.float64) * 4 / 2) * 2
    W2 = np.round(snn["w2learned"].astype(np.float64) * 4 / 2) * 2

    def loihi(ws):
        s, v, u = O.loihi_get_spikes((ws * Ts).astype(np.float32), 0, theta, 1024, 128, 1)
        return s / Ts, v

    sH, vH = loihi(W1 @ x.astype(np.float64))
    sH = O.shift(sH, 1, 1)
    sO, vO = loihi(W2 @ sH.astype(np.float64))
    sO = O.shift(sO, 1, 1)
    assert np.array_equal(sH, raster_from_aer(chip["hiddenSpikes"], 25, Ns, Ts, 1 / Ts, time_first=False))
    assert len(chip["hiddenSpikes"]) == 639
    assert np.array_equal(np.nonzero(sO[0])[0], np.array([57, 60]))
    assert np.array_equal(vH[24, :-1], chip["hiddenVoltage24"].astype(np.float32))
    assert np.array_equal(vH[23, :-1], chip["hiddenVoltage23"].astype(np.float32))
    assert np.array_equal(vO[0, :-1], chip["outputVoltage"].astype(np.float32))


def test_loihi_impulse_response_is_twice_the_psp_kernel():
    w = np.zeros((1, 130), np.float32)
    w[0, 1] = 2
    s, v, u = O.loihi_get_spikes(w, 0, 80 * 64, 1024, 128, 1)
    psp = 2 * np.array(loihiPspKernel(1024, 128, 0))
    assert not s.any()
    assert np.array_equal(v[0, 1:1 + len(psp)], psp.astype(np.float32))


# ------------------------------------------------------------------------------------------
# joint forward + backward: golden weight gradients of the 250-25-1 network
# ------------------------------------------------------------------------------------------
def test_joint_gradients_golden():
    """spike(psp(fc(x))) twice, spikeTime loss against spikeOut.txt, tauRho = 0.1, full refractory
    kernel: d loss / d W must equal gradW{1,2}Initial.txt (criterion of the reference's
    test_slayer003: ||diff|| / size < 1e-4).  Backward is assembled by hand from the oracle's
    corr and spike_bwd, so conv, corr, spike and spike_bwd are pinned together."""
    snn = golden("snn_250_25_1.npz")
    Ts, Ns, theta, tauRho, scaleRho = 0.1, 500, 10.0, 0.1, 1.0
    srm = np.array(alphaKernel(1.0, Ts, 50), dtype=np.float32)
    ref = np.array(alphaKernel(1.0, Ts, 50, mult=-20, EPSILON=0.0001), dtype=np.float32)
    x = raster_from_aer(snn["spikeIn"], 250, Ns, Ts, 1 / Ts)
    des = raster_from_aer(snn["spikeOut"], 1, Ns, Ts, 1 / Ts)
    W1, W2 = snn["w1Initial"], snn["w2Initial"]

    z1 = (W1.astype(np.float64) @ x).astype(np.float32)
    s1, u1 = O.get_spikes(O.conv(z1, srm, Ts).reshape(1, 25, 1, 1, Ns), ref, theta, Ts)
    s1, u1 = s1.reshape(25, Ns), u1.reshape(25, Ns)
    z2 = (W2.astype(np.float64) @ s1).astype(np.float32)
    s2, u2 = O.get_spikes(O.conv(z2, srm, Ts).reshape(1, 1, 1, 1, Ns), ref, theta, Ts)
    s2, u2 = s2.reshape(1, Ns), u2.reshape(1, Ns)

    err = O.conv(s2 - des, srm, Ts)                       # loss = 1/2 sum(err^2) Ts
    g_s2 = O.corr(err * Ts, srm, Ts)
    g_z2 = O.corr(O.spike_bwd(g_s2, u2, theta, tauRho * theta, scaleRho), srm, Ts)
    gW2 = g_z2.astype(np.float64) @ s1.T.astype(np.float64)
    g_s1 = W2.T.astype(np.float64) @ g_z2
    g_z1 = O.corr(O.spike_bwd(g_s1.astype(np.float32), u1, theta, tauRho * theta, scaleRho), srm, Ts)
    gW1 = g_z1.astype(np.float64) @ x.T.astype(np.float64)

    assert np.linalg.norm(gW2 - snn["gradW2Initial"]) / gW2.size < 1e-4
    assert np.linalg.norm(gW1 - snn["gradW1Initial"]) / gW1.size < 1e-4
    assert np.linalg.norm(snn["gradW1Initial"]) / gW1.size > 1e-3   # the criterion is not vacuous


# ------------------------------------------------------------------------ spike event files
def _spike_events():
    return np.load(os.path.join(os.path.dirname(__file__), "golden", "spike_events.npz"))


def test_event_decoding_matches_reference_sample():
    """NMNISTsmall/1.bs2 against the reference's listing of the same sample
    (input_validate/1_raw_spikes.csv: x, y, p one-based, t in us)."""
    g = _spike_events()
    x, y, p, t = O.decode_events(g["nmnist_bs2"], 2)
    raw = g["nmnist_raw"]
    assert x.size == raw.shape[0] == 4681
    assert np.array_equal(x, raw[:, 0] - 1) and np.array_equal(y, raw[:, 1] - 1)
    assert np.array_equal(p, raw[:, 2] - 1) and np.array_equal(t, raw[:, 3])


def test_event_decoding_bit_fields():
    """All three layouts against the shifts and masks written out with numpy integer arithmetic."""
    g = _spike_events()
    b = g["ntidigits_bs1"].astype(np.int64).reshape(-1, 5)
    x, y, p, t = O.decode_events(g["ntidigits_bs1"], 1)
    assert np.array_equal(x, (b[:, 0] << 8) | b[:, 1]) and not y.any()
    assert np.array_equal(p, b[:, 2] >> 7)
    assert np.array_equal(t, ((b[:, 2] << 16) | (b[:, 3] << 8) | b[:, 4]) & 0x7FFFFF)
    assert x.max() < 64 and np.all(np.diff(t) >= 0)            # 64 cochlea channels, sorted in time
    b = g["sample_bs3"].astype(np.int64).reshape(-1, 7)
    x, y, p, t = O.decode_events(g["sample_bs3"], 3)
    assert np.array_equal(x, (b[:, 0] << 4) | (b[:, 1] >> 4))
    assert np.array_equal(y, b[:, 2] | ((b[:, 1] & 0x0F) << 8))
    assert np.array_equal(p, b[:, 3]) and np.array_equal(t, (b[:, 4] << 16) | (b[:, 5] << 8) | b[:, 6])
    assert np.all(np.diff(t) >= 0)


def test_event_binning_matches_reference_rasters():
    """The reference's binned rasters of the NMNIST sample (1 ms and 2 ms bins; they were binned by
    truncation, so the times are moved to the start of their bin first): pins layout, validity and
    value of the binning."""
    g = _spike_events()
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "nmnist_response.npz"))
    x, y, p, t = O.decode_events(g["nmnist_bs2"], 2)
    for Ts, key in ((1, "binned"), (2, "binned_ts2")):
        shape = tuple(gold[key + "_shape"])
        raster = np.zeros(shape, np.float32)
        raster[gold[key + "_events"][:, 0], gold[key + "_events"][:, 1]] = gold[key + "_values"]
        got = O.bin_events(np.zeros((2, 34, 34, shape[1]), np.float32), x, y, p - p.min(),
                           np.floor(t / 1000 / Ts) * Ts, Ts)
        assert np.array_equal(got.reshape(shape), raster)


def test_event_binning_rounding_and_modes():
    """Bin = numpy.round(t / Ts) (half to even) minus the shift; OR stores 1/Ts; SUM adds it once per
    occupied bin, which is what numpy's indexed += does."""
    rng = np.random.default_rng(2)
    n, (C, H, W, T), Ts, shift = 4000, (2, 5, 6, 40), 1.5, 3
    x, y, p = rng.integers(-1, W + 2, n), rng.integers(-1, H + 2, n), rng.integers(0, C + 1, n)
    t = rng.random(n) * 80 - 3
    t[::4] = (np.floor(t[::4] / Ts) + 0.5) * Ts                 # exactly half way
    base = rng.standard_normal((C, H, W, T)).astype(np.float32)
    tb = np.round(t / Ts).astype(int) - shift
    ok = (x >= 0) & (x < W) & (y >= 0) & (y < H) & (p >= 0) & (p < C) & (tb >= 0) & (tb < T)
    for mode in ("OR", "SUM"):
        ref = base.copy()
        if mode == "OR":
            ref[p[ok], y[ok], x[ok], tb[ok]] = 1 / Ts
        else:
            ref[p[ok], y[ok], x[ok], tb[ok]] += 1 / Ts
        got = O.bin_events(base, x, y, p, t, Ts, shift, mode)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


# ------------------------------------------------------------------------ per-timestep synapses
SYNAPSE_CASES = [
    # N, C, H, W, T, O, (KH, KW), stride, padding, dilation, groups
    (2, 4, 9, 8, 5, 6, (3, 3), 1, 1, 1, 1),
    (1, 4, 10, 11, 3, 8, (3, 2), (2, 1), (1, 0), (1, 2), 2),
    (2, 1, 8, 8, 4, 1, (2, 2), 2, 0, 1, 1),
    (1, 6, 7, 7, 2, 6, (3, 3), 2, 2, 2, 3),
    (1, 2, 4, 4, 3, 2, (5, 5), 1, 0, 1, 1),        # the filter does not fit: empty output
]


@pytest.mark.parametrize("case", SYNAPSE_CASES)
def test_synapse_oracle_matches_torch_conv3d(case):
    """The oracle's synapse and both gradients against F.conv3d with a (KH, KW, 1) kernel and its
    autograd on the CPU - the very call the reference's layers make (src/slayer.py:499-507)."""
    N, C, H, W, T, Oc, K, s, p, d, g = case
    rng = np.random.default_rng(0)
    x = rng.standard_normal((N, C, H, W, T)).astype(np.float32)
    w = rng.standard_normal((Oc, C // g, K[0], K[1])).astype(np.float32)
    tup = lambda v: (v, v) if isinstance(v, int) else tuple(v)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w[..., None], dtype=torch.float64, requires_grad=True)
    if O.synapse_geom(x.shape, w.shape, s, p, d, g)[1][2] == 0:
        assert O.synapse_conv(x, w, s, p, d, g).size == 0
        return
    y = F.conv3d(xt, wt, None, tup(s) + (1,), tup(p) + (0,), tup(d) + (1,), g)
    yo = O.synapse_conv(x, w, s, p, d, g)
    assert yo.shape == tuple(y.shape)
    assert rel_err(yo, y.detach().numpy()) < 1e-6
    go = rng.standard_normal(yo.shape).astype(np.float32)
    y.backward(torch.tensor(go, dtype=torch.float64))
    assert rel_err(O.synapse_conv_grad_input(go, w, x.shape, s, p, d, g), xt.grad.numpy()) < 1e-6
    assert rel_err(O.synapse_conv_grad_weight(go, x, w.shape, s, p, d, g), wt.grad.numpy()[..., 0]) < 1e-6


def test_synapse_oracle_shift_and_add():
    """The constructions of the reference's own tests: convolution as a sum of shifted, weighted
    copies (test/test_slayer007.py:36-48), pooling as the sum of the four window positions (:60-66),
    transposed convolution as every input sample spread over its window (test/test_slayer013.py)."""
    rng = np.random.default_rng(1)
    N, C, H, W, D, K = 2, 3, 9, 10, 4, 5
    x = rng.standard_normal((N, C, H, W, D)).astype(np.float32)
    w = rng.standard_normal((1, C, K, K)).astype(np.float32)
    ref = np.zeros((N, 1, H - K + 1, W - K + 1, D))
    for i in range(K):
        for j in range(K):
            for k in range(C):
                ref[:, 0] += w[0, k, j, i].astype(np.float64) * x[:, k, j:H - K + 1 + j, i:W - K + 1 + i, :]
    assert rel_err(O.synapse_conv(x, w), ref) < 1e-6
    x = rng.standard_normal((2, 1, 8, 6, 4)).astype(np.float32)
    ones = np.full((1, 1, 2, 2), 11.0, np.float32)
    ref = (x[:, :, 0::2, 0::2] + x[:, :, 0::2, 1::2] + x[:, :, 1::2, 0::2] + x[:, :, 1::2, 1::2]) * 11.0
    assert rel_err(O.synapse_conv(x, ones, 2), ref) < 1e-6
    Cin, Cout, K, H, W = 2, 3, 3, 4, 5
    x = rng.standard_normal((1, Cin, H, W, 3)).astype(np.float32)
    w = rng.standard_normal((Cin, Cout, K, K)).astype(np.float32)
    ref = np.zeros((1, Cout, H + K - 1, W + K - 1, 3))
    for i in range(K):
        for j in range(K):
            for m in range(Cin):
                for k in range(Cout):
                    ref[:, k, i:i + H, j:j + W, :] += w[m, k, i, j].astype(np.float64) * x[:, m]
    assert rel_err(O.synapse_conv_grad_input(x, w, ref.shape), ref) < 1e-6

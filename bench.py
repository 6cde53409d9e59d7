#!/usr/bin/env python3
"""Benchmark of SLAYER's temporal kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

One step = one pass of the hot path over one batch of synthetic input, forward and backward:

    forward : a = psp(spikes)  (conv, 77-tap SRM kernel)   s = spike(u)   d = delayShift(s, 1)
    backward: gd = shift(g, -1)   gs = spikeBackward(gd, u')   ga = corr(gs, SRM kernel)

on the NMNIST-CNN-shaped activation tensor (12, 16, 34, 34, 300), fp32, all inputs resident in
HBM.  The spike kernel updates its input in place, so each step works on its own pre-made copy
of the membrane potential (made before the timed region).  Prints ONE JSON line:
neuron-timesteps/s of the chain, the HBM roofline of the dominant kernel (HIP events around its
launches inside the timed region, on the launch stream) and the CPU oracle timed on the host
cores beside it.
"""
import argparse
import json
import os
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

SHAPE = (12, 16, 34, 34, 300)
HBM_PEAK_GBS = 8000.0                     # MI355X HBM3E, published
FP32_PEAK_TFLOPS = 157.3                  # MI355X FP32, published: vector (with packed FP32; scalar FMAs: 78.6) and matrix alike
SRM_TAPS = 77
# algorithmic bytes per neuron-timestep (fp32 tensors read + written once)
AB = {"psp_conv": 8, "spike": 12, "shift": 8, "shift_bwd": 8, "spike_bwd": 12, "psp_corr": 8}
# HBM bytes per launch on SHAPE measured with the FETCH_SIZE and WRITE_SIZE hardware counters
# (rocprofv3 --pmc, one counter per run, scaled by the reading of a plain copy of known size):
# profiles/hbm_traffic_counters.json holds the figures, profiles/hbm_traffic_counters.txt the commands
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_counters.json")


def measured_traffic(op):
    """HBM bytes per launch of `op` on SHAPE from the committed counter run, and where they come from (the file
    names the commit of the library the counters were read on)."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f)
        return rec["bytes_per_launch"].get(op), {"file": "profiles/hbm_traffic_counters.json", "library_commit": rec.get("commit"),
                                                 "kernel": rec.get("kernels", {}).get(op)}
    except (OSError, ValueError, KeyError):
        return None, None
KERNEL_OF = {"psp_conv": "slayer::alpha_psp_kernel<true, 4, 0, true> (conv with the alpha kernel as a recursion over time)",
             "spike": "slayer::spike_tile_kernel<12, 1, 12, 8>",
             "shift": "slayer::shift_vec_kernel<0>", "shift_bwd": "slayer::shift_vec_kernel<0>",
             "spike_bwd": "slayer::spike_bwd_vec_kernel",
             "psp_corr": "slayer::alpha_psp_kernel<false, 4, 0, true> (corr with the alpha kernel as a recursion over time)"}


def neuron_params():
    return {"theta": 10.0, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2.0, "tauRho": 1.0, "scaleRho": 1.0}


def make_inputs(shape, device, seed=0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    spikes = (torch.rand(shape, generator=g) < 0.02).float()
    u0 = torch.randn(shape, generator=g) * 5.0
    g1 = torch.Generator(device="cpu").manual_seed(seed + 1)
    grad = torch.randn(shape, generator=g1)
    return spikes.to(device), u0.to(device), grad.to(device)


def cpu_baseline(shape, srm, ref, params, rows_fraction=1):
    """The CPU oracle on a bounded sample of the same workload (every rows_fraction-th batch
    slice), all host threads."""
    from oracle import oracle as O
    threads = O.max_threads()
    O.set_threads(threads)
    rows = (shape[0] * shape[1] * shape[2] * shape[3]) // rows_fraction
    rows -= rows % (shape[2] * shape[3])
    sub = (1, rows // (shape[2] * shape[3]), shape[2], shape[3], shape[4])
    rng = np.random.default_rng(0)
    spikes = (rng.random(sub) < 0.02).astype(np.float32)
    u0 = (rng.standard_normal(sub) * 5).astype(np.float32)
    grad = rng.standard_normal(sub).astype(np.float32)
    theta, tau, scale = params["theta"], params["tauRho"] * params["theta"], params["scaleRho"]
    times = []
    began = time.perf_counter()
    while len(times) < 3 or (time.perf_counter() - began < 10.0 and len(times) < 200):   # about 10 s of CPU work
        t0 = time.perf_counter()
        O.conv(spikes, srm, 1.0)
        s, u = O.get_spikes(u0, ref, theta, 1.0)
        O.shift(s, 1.0, 1.0)
        gd = O.shift(grad, -1.0, 1.0)
        gs = O.spike_bwd(gd, u, theta, tau, scale)
        O.corr(gs, srm, 1.0)
        times.append(time.perf_counter() - t0)
    best = sorted(times)[len(times) // 2]
    O.set_threads(1)
    return {"value": spikes.size / best, "unit": "neuron-timesteps/s", "cores": threads, "kind": "port",
            "sample": "oracle chain (conv77+spike+shift, shift+spike_bwd+corr77) on %s, median of %d passes, %.2f s each"
                      % (str(sub), len(times), best)}


def cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_plumbing_baseline(srm, ref, params):
    """The reference's own CPU-runnable case, timed on the host cores: Bernoulli(0.02) spikes (4, 2, 34, 34, 300),
    dense 2312 -> 512 as torch's conv3d with a (34, 34, 1) kernel (src/slayer.py:393-449), the PSP as a left-padded
    conv3d with the flipped SRM kernel like pspLayer (src/slayer.py:760-791), torch on all host threads; then the
    threshold / refractory loop by the CPU oracle.  Reported beside the GPU figures, not a target."""
    import torch.nn.functional as F
    from oracle import oracle as O
    threads = os.cpu_count() or 1
    old = torch.get_num_threads()
    torch.set_num_threads(threads)
    O.set_threads(O.max_threads())
    try:
        g = torch.Generator().manual_seed(0)
        x = (torch.rand((4, 2, 34, 34, 300), generator=g) < 0.02).float()
        w = torch.randn((512, 2, 34, 34, 1), generator=g) * 100.0      # N(0,1) * scale 100, as the case is stated
        k = torch.from_numpy(srm[::-1].copy()).reshape(1, 1, 1, 1, -1)
        times = {"dense_conv3d": [], "psp_conv3d": [], "spike_oracle": []}
        for _ in range(6):
            t0 = time.perf_counter()
            a = F.conv3d(x, w)                                               # (4, 512, 1, 1, 300)
            t1 = time.perf_counter()
            u = F.conv3d(F.pad(a.reshape(4, 1, 512, 1, 300), (len(srm) - 1, 0)), k).reshape(a.shape)
            t2 = time.perf_counter()
            O.get_spikes(u.numpy().copy(), ref, params["theta"], 1.0)
            t3 = time.perf_counter()
            for name, dt in zip(times, (t1 - t0, t2 - t1, t3 - t2)):
                times[name].append(dt)
        med = {n: float(np.median(v[1:])) for n, v in times.items()}
        total = sum(med.values())
        return {"value": u.numel() / total, "unit": "neuron-timesteps/s", "cores": threads, "kind": "port",
                "sample": "CPU plumbing case: torch conv3d dense 2312->512 + pspLayer-style conv3d PSP (77 taps) + oracle "
                          "spike loop on (4, 2, 34, 34, 300) -> (4, 512, 1, 1, 300), median of 5 passes",
                "seconds": med, "torch_threads": torch.get_num_threads()}
    finally:
        torch.set_num_threads(old)
        O.set_threads(1)


def copy_ceiling(x):
    """What plain copies of the benchmark tensor reach on this box (read + written bytes per second):
    the runtime's device-to-device copy and this library's zero-delay shift (one 16-byte vector
    per lane, streaming policy)."""
    from slayerpytorch_amd import slayerCuda
    y = torch.empty_like(x)

    def timed(fn):
        ts = []
        for i in range(10):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            fn()
            b.record()
            torch.cuda.synchronize()
            if i >= 3:
                ts.append(a.elapsed_time(b) * 1e-3)
        return float(np.median(ts))

    nbytes = 2 * x.numel() * 4
    return {"unit": "GB/s", "device_to_device_copy": nbytes / timed(lambda: y.copy_(x)) / 1e9,
            "zero_delay_shift_kernel": nbytes / timed(lambda: slayerCuda.shift(x, 0.0, 1.0)) / 1e9}


def flip_rate(device, srm_t, ref_t, params):
    """Part of the CPU leg.  Fraction of spike samples that differ between the GPU chain psp -> scale -> spike and the
    CPU oracle chain run with separately rounded multiply and add (the only difference between
    the two is the fp32 rounding of the filter sum upstream of the threshold)."""
    from oracle import oracle as O
    from slayerpytorch_amd import slayerCuda
    rng = np.random.default_rng(0)
    shape = (2, 16, 34, 34, 300)
    spikes = (rng.random(shape) < 0.02).astype(np.float32)
    gain = np.float32(9.0)           # puts about 2 % of the samples above threshold
    a = slayerCuda.pspAlpha(torch.from_numpy(spikes).to(device), srm_t, params["tauSr"], 1.0, 1.0, True) * float(gain)
    s_gpu = slayerCuda.getSpikes(a.contiguous(), ref_t, params["theta"], 1.0).cpu().numpy()
    a_cpu = O.conv(spikes, srm_t.cpu().numpy(), 1.0, fused=False) * gain
    s_cpu, _ = O.get_spikes(a_cpu, ref_t.cpu().numpy(), params["theta"], 1.0)
    return float((s_gpu != s_cpu).mean()), float((s_cpu != 0).mean())


def layer_flip_rate(device, srm_t, ref_t, params):
    """Part of the CPU leg.  The same for a whole layer of the NMNIST CNN: spike(conv 2->16 5x5 (psp(x))) on
    (4, 2, 34, 34, 300) input spikes, the GPU chain (psp as the layers run it, fp32 synapse kernel, spike kernel)
    against the CPU oracle chain (separately rounded psp, synapse accumulated in double, spike loop)."""
    from oracle import oracle as O
    from slayerpytorch_amd import slayerCuda, synapse
    rng = np.random.default_rng(1)
    x = (rng.random((4, 2, 34, 34, 300)) < 0.02).astype(np.float32)
    w = (rng.standard_normal((16, 2, 5, 5)) * 1.5).astype(np.float32)     # about 3 % of the output samples spike
    a = slayerCuda.pspAlpha(torch.from_numpy(x).to(device), srm_t, params["tauSr"], 1.0, 1.0, True)
    u = synapse.conv(a, torch.from_numpy(w).to(device), 1, 1)
    s_gpu = slayerCuda.getSpikes(u, ref_t, params["theta"], 1.0).cpu().numpy()
    threads = O.lib().oracle_get_threads()
    O.set_threads(O.max_threads())
    try:
        u_cpu = O.synapse_conv(O.conv(x, srm_t.cpu().numpy(), 1.0, fused=False), w, 1, 1)
        s_cpu, _ = O.get_spikes(u_cpu, ref_t.cpu().numpy(), params["theta"], 1.0)
    finally:
        O.set_threads(threads)
    return float((s_gpu != s_cpu).mean()), float((s_cpu != 0).mean())


def mlp_row(device, timed):
    """One training step (without the optimiser) of the 2312-512-10 MLP on (12, 2, 34, 34, 350) input
    spikes at p = 0.015, layer ordering spike(psp(fc(x))), spike-time loss against a random target
    train; both the separate calls and the fused pspSpike call."""
    import slayerpytorch_amd as snn
    params = neuron_params()
    sim = {"Ts": 1.0, "tSample": 350}
    net = {"neuron": params, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}
    layer = snn.layer(params, sim).to(device)
    error = snn.loss(net).to(device)
    torch.manual_seed(0)
    fc1, fc2 = layer.dense((34, 34, 2), 512).to(device), layer.dense(512, 10).to(device)
    g = torch.Generator(device="cpu").manual_seed(3)
    x = (torch.rand((12, 2, 34, 34, 350), generator=g) < 0.015).float().to(device)
    target = (torch.rand((12, 10, 1, 1, 350), generator=g) < 0.01).float().to(device)

    def step(fused):
        if fused:
            s2 = layer.pspSpike(fc2(layer.pspSpike(fc1(x))))
        else:
            s2 = layer.spike(layer.psp(fc2(layer.spike(layer.psp(fc1(x))))))
        loss = error.spikeTime(s2, target)
        loss.backward()
        fc1.weight.grad = None
        fc2.weight.grad = None

    two = timed(lambda: step(False))
    one = timed(lambda: step(True))
    row = {"op": "nmnist_mlp_2312_512_10_fwd_loss_bwd", "shape": [12, 2, 34, 34, 350], "us": one * 1e6,
           "us_with_separate_psp_and_spike_calls": two * 1e6, "samples_per_s": 12 / min(one, two)}
    # The step is launch-bound (about 25 short kernels): captured once in a HIP graph and replayed.  The
    # library's entry points only enqueue on the stream they are given, so they can be captured as they are.
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            step(False)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        step(False)
    row["us_replayed_from_hip_graph"] = timed(graph.replay) * 1e6
    return row


def scale_weights_to_rate(weight, rate, target=0.04):
    """Scales a random weight tensor in place until ``rate()`` (the fraction of output samples that
    are spikes) is within 25 % of ``target``: random weights at the default scale leave a layer
    silent or saturated, a trained network fires a few per cent of the time."""
    with torch.no_grad():
        for _ in range(16):
            r = rate()
            if 0.75 * target <= r <= 1.25 * target:
                break
            weight.mul_(min(3.0, max(0.3, (target / max(r, 1e-4)) ** 0.7)))


def delay_mlp_row(device, timed):
    """One training step (without the optimiser) of the long-sequence delay network: 200 input neurons
    with Poisson spikes at 0.005 per step, batch 64, T = 2000, dense 200 -> 256 -> 200 with a learnable
    axonal delay per neuron (U[0, 62]) after every layer, SRM tauSr = tauRef = 1, spike-time loss against
    a random raster at p = 0.01; layer ordering delay(spike(psp(fc(x))))."""
    import slayerpytorch_amd as snn
    params = {"type": "SRMALPHA", "theta": 10, "tauSr": 1.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    sim = {"Ts": 1.0, "tSample": 2000}
    net = {"neuron": params, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}
    layer = snn.layer(params, sim).to(device)
    error = snn.loss(net).to(device)
    torch.manual_seed(0)
    fc1, fc2 = layer.dense(200, 256).to(device), layer.dense(256, 200).to(device)
    d1, d2 = layer.delay(256).to(device), layer.delay(200).to(device)
    with torch.no_grad():
        d1.delay.mul_(62.0)
        d2.delay.mul_(62.0)
    g = torch.Generator(device="cpu").manual_seed(7)
    x = (torch.rand((64, 200, 1, 1, 2000), generator=g) < 0.005).float().to(device)
    target = (torch.rand((64, 200, 1, 1, 2000), generator=g) < 0.01).float().to(device)
    rates = []
    with torch.no_grad():
        scale_weights_to_rate(fc1.weight, lambda: float(layer.spike(layer.psp(fc1(x))).mean()))
        s1 = d1(layer.spike(layer.psp(fc1(x))))
        scale_weights_to_rate(fc2.weight, lambda: float(layer.spike(layer.psp(fc2(s1))).mean()))

    def step(fused=True):
        if fused:   # delay(spike(u)) from one kernel each way (the spikes are shifted while they are stored)
            s1 = layer.spikeDelayed(layer.psp(fc1(x)), d1)
            s2 = layer.spikeDelayed(layer.psp(fc2(s1)), d2)
        else:
            s1 = d1(layer.spike(layer.psp(fc1(x))))
            s2 = d2(layer.spike(layer.psp(fc2(s1))))
        del rates[:]
        rates.extend((s1, s2))
        error.spikeTime(s2, target).backward()
        for m in (fc1, fc2):
            m.weight.grad = None
        for m in (d1, d2):
            m.delay.grad = None

    two = timed(lambda: step(False))
    t = timed(step)
    return {"op": "delay_mlp_200_256_200_fwd_loss_bwd", "shape": [64, 200, 1, 1, 2000], "us": t * 1e6,
            "us_with_separate_spike_and_delay_calls": two * 1e6,
            "samples_per_s": 64 / t, "spike_rate_per_layer": [round(float(r.detach().mean()), 4) for r in rates]}


def cnn_row(device, timed):
    """One training step (without the optimiser) of the NMNIST CNN of the reference's example
    (example/03_NMNIST_CNN/nmnistCNN.py:47-62: conv 2->16 5x5, pool 2, conv 16->32 3x3, pool 2,
    conv 32->64 3x3, dense 4096->10, every layer as spike(synapse(psp(x)))) on (12, 2, 34, 34, 300)
    input spikes at p = 0.02 with a spike-time loss against a random target train.  Random weights,
    scaled per layer to a spike rate of about 4 % (reported in the row)."""
    import slayerpytorch_amd as snn
    params = neuron_params()
    sim = {"Ts": 1.0, "tSample": 300}
    net = {"neuron": params, "simulation": sim, "training": {"error": {"type": "SpikeTime"}}}
    layer = snn.layer(params, sim).to(device)
    error = snn.loss(net).to(device)
    torch.manual_seed(0)
    conv1, conv2, conv3 = layer.conv(2, 16, 5, padding=1), layer.conv(16, 32, 3, padding=1), layer.conv(32, 64, 3, padding=1)
    pool1, pool2, fc1 = layer.pool(2), layer.pool(2), layer.dense((8, 8, 64), 10)
    mods = [m.to(device) for m in (conv1, conv2, conv3, pool1, pool2, fc1)]
    g = torch.Generator(device="cpu").manual_seed(5)
    x = (torch.rand((12, 2, 34, 34, 300), generator=g) < 0.02).float().to(device)
    target = (torch.rand((12, 10, 1, 1, 300), generator=g) < 0.01).float().to(device)
    rates = []
    # random weights scaled, front to back, until about 4 % of a trainable layer's output samples are spikes
    with torch.no_grad():
        s = x
        for syn in (conv1, pool1, conv2, pool2, conv3, fc1):
            a = layer.psp(s)
            if syn.weight.requires_grad:
                scale_weights_to_rate(syn.weight, lambda: float(layer.spike(syn(a)).mean()))
            s = layer.spike(syn(a))

    def step():
        s = x
        for syn in (conv1, pool1, conv2, pool2, conv3, fc1):
            s = layer.spike(syn(layer.psp(s)))
        error.spikeTime(s, target).backward()
        for m in mods:
            m.weight.grad = None

    with torch.no_grad():
        s = x
        for syn in (conv1, pool1, conv2, pool2, conv3, fc1):
            s = layer.spike(syn(layer.psp(s)))
            rates.append(round(float(s.mean()), 4))
    t = timed(step)
    row = {"op": "nmnist_cnn_fwd_loss_bwd", "shape": [12, 2, 34, 34, 300], "us": t * 1e6, "samples_per_s": 12 / t,
           "spike_rate_per_layer": rates}
    # the same step with the backward passes of every hidden layer's spike function and of the next layer's PSP filter
    # as the two kernels they are in the reference (the default sends psp's gradient past the spike function in one kernel)
    from slayerpytorch_amd import slayer as slayer_module
    paired = slayer_module.PAIR_SPIKE_PSP
    slayer_module.PAIR_SPIKE_PSP = False
    try:
        row["us_with_spike_and_psp_backward_apart"] = timed(step) * 1e6
    finally:
        slayer_module.PAIR_SPIKE_PSP = paired
    return row


SYNAPSE_LAYERS = (
    # name, input shape (N, C, H, W, T), weight shape, stride, padding, input spike density
    ("conv 2->16 5x5", (12, 2, 34, 34, 300), (16, 2, 5, 5), 1, 1, 0.02),
    ("pool 2x2 on 16x32x32", (12, 1, 16 * 32, 32, 300), (1, 1, 2, 2), 2, 0, 0.05),
    ("conv 16->32 3x3", (12, 16, 16, 16, 300), (32, 16, 3, 3), 1, 1, 0.05),
    ("pool 2x2 on 32x16x16", (12, 1, 32 * 16, 16, 300), (1, 1, 2, 2), 2, 0, 0.05),
    ("conv 32->64 3x3", (12, 32, 8, 8, 300), (64, 32, 3, 3), 1, 1, 0.05),
)


def synapse_rows(device, timed):
    """The per-timestep synapse kernels on the layer shapes of the NMNIST CNN: forward, input
    gradient and weight gradient, with the fp32 rate (2 flop per multiply-add) and the fraction of
    HBM peak that the tensors each kernel must move at least once amount to."""
    from slayerpytorch_amd import synapse
    g = torch.Generator(device="cpu").manual_seed(9)
    rows = []
    for name, xs, ws, stride, pad, density in SYNAPSE_LAYERS:
        x = (torch.rand(xs, generator=g) < density).float().to(device)
        w = torch.randn(ws, generator=g).to(device)
        y = synapse.conv(x, w, stride, pad)
        gy = torch.randn(y.shape, generator=g).to(device)
        flop = 2.0 * y.numel() * ws[1] * ws[2] * ws[3]
        nbytes = 4.0 * (x.numel() + y.numel())
        for op, fn in (("forward", lambda: synapse.conv(x, w, stride, pad)),
                       ("grad_input", lambda: synapse.convGradInput(gy, w, x.shape, stride, pad)),
                       ("grad_weight", lambda: synapse.convGradWeight(gy, x, w.shape, stride, pad))):
            if op == "grad_weight" and name.startswith("pool"):
                continue            # pooling weights are constants
            t = timed(fn)
            rows.append({"op": "synapse " + op + " " + name, "shape": list(xs), "us": t * 1e6,
                         "tflops_fp32": flop / t / 1e12, "hbm_frac": nbytes / t / 1e9 / HBM_PEAK_GBS})
        del x, w, y, gy
    return rows


def loihi_cnn_row(device, timed):
    """Inference of the Loihi gesture network of the reference's example
    (exampleLoihi/03_IBMGesture/ibmGestureTrain.py:44-79, without dropout) on (8, 2, 128, 128, 300) input
    spikes at p = 0.01: pool 4, conv 2->16 5x5, pool 2, conv 16->32 3x3, pool 2, dense 2048->512->11, weights
    quantised to even integers, every layer as delayShift(spikeLoihi(synapse(x)), 1) with the shift fused
    into the neuron kernel; no autograd."""
    import slayerpytorch_amd as snn
    desc = {"type": "LOIHI", "vThMant": 80, "vDecay": 128, "iDecay": 1024, "refDelay": 1, "wgtExp": 0,
            "tauRho": 1, "scaleRho": 1}
    layer = snn.loihi(desc, {"Ts": 1, "tSample": 300}).to(device)
    torch.manual_seed(0)
    mods = [layer.pool(4), layer.conv(2, 16, 5, padding=2, weightScale=10), layer.pool(2),
            layer.conv(16, 32, 3, padding=1, weightScale=50), layer.pool(2), layer.dense(8 * 8 * 32, 512),
            layer.dense(512, 11)]
    mods = [m.to(device) for m in mods]
    g = torch.Generator(device="cpu").manual_seed(6)
    x = (torch.rand((8, 2, 128, 128, 300), generator=g) < 0.01).float().to(device)
    rates = []

    def step():
        del rates[:]
        with torch.no_grad():
            s = x
            for k, syn in enumerate(mods):
                if k == 5:
                    s = s.reshape(s.shape[0], -1, 1, 1, s.shape[-1])
                s = layer.spikeLoihi(syn(s), delay=1)
                rates.append(s)

    t = timed(step)
    row = {"op": "loihi_gesture_cnn_inference", "shape": [8, 2, 128, 128, 300], "us": t * 1e6, "samples_per_s": 8 / t,
           "spike_rate_per_layer": [round(float(r.mean()), 4) for r in rates]}

    # the same network trained: forward with autograd, spike-time loss against a random target, backward
    # (surrogate gradient fused into the 110-tap correlation, quantised weights with straight-through gradient)
    error = snn.loss({"neuron": desc, "simulation": {"Ts": 1, "tSample": 300},
                      "training": {"error": {"type": "SpikeTime"}}}, snn.loihi).to(device)
    target = (torch.rand((8, 11, 1, 1, 300), generator=g) < 0.02).float().to(device)

    def train_step():
        s = x
        for k, syn in enumerate(mods):
            if k == 5:
                s = s.reshape(s.shape[0], -1, 1, 1, s.shape[-1])
            s = layer.spikeLoihi(syn(s), delay=1)
        error.spikeTime(s, target).backward()
        for m in mods:
            m.weight.grad = None

    row["us_training_step"] = timed(train_step) * 1e6
    return row


def event_row(device, timed, cpu_leg):
    """A batch of 12 NMNIST-sized samples (5000 events each, the 5-byte layout of the .bs2 files)
    to a (12, 2, 34, 34, 300) spike tensor: file bytes uploaded and decoded + binned by one kernel
    into a zeroed tensor.  With the CPU leg: against the host sequence the reference's data loaders run
    (decode and bin with the CPU oracle, then upload the dense tensor), as part of the CPU baseline."""
    import slayerpytorch_amd as snn
    rng = np.random.default_rng(4)
    n, shape = 5000, (12, 2, 34, 34, 300)
    raws = []
    for _ in range(shape[0]):
        x, y, p = rng.integers(0, 34, n), rng.integers(0, 34, n), rng.integers(0, 2, n)
        t = np.sort(rng.integers(0, 300000, n))
        b = np.zeros((n, 5), dtype=np.uint8)
        b[:, 0], b[:, 1], b[:, 2] = x, y, ((t >> 16) & 0x7F) | (p << 7)
        b[:, 3], b[:, 4] = (t >> 8) & 0xFF, t & 0xFF
        raws.append(b.reshape(-1))
    events = [snn.io.event._fromBytes(r, 2) for r in raws]

    def on_device():
        return snn.io.toSpikeTensorBatch(events, torch.zeros(shape, device=device), 1.0)

    def on_host():
        from oracle import oracle
        out = np.zeros(shape, dtype=np.float32)
        for i, r in enumerate(raws):
            x, y, p, t = oracle.decode_events(r, 2)
            out[i] = oracle.bin_events(out[i], x, y, p - p.min(), t / 1000, 1.0)
        return torch.from_numpy(out).to(device)

    dev_t = timed(on_device)
    row = {"op": "event files -> spike tensor (decode + bin, 12 x 5000 events)", "shape": list(shape),
           "us": dev_t * 1e6, "events_per_s": shape[0] * n / dev_t}
    if cpu_leg:
        row["us_host_decode_bin_and_dense_upload"] = timed(on_host) * 1e6
        row["identical_to_host_result"] = bool(torch.equal(on_device(), on_host()))
    return row


def other_rows(device, cpu_leg=False):
    """Quick per-op measurements of the scope rows that are not part of the headline chain, each on
    the largest tensor its benchmark configuration gives it (kernel rows: median of 7 event-timed passes of 8
    launches back to back; network steps: median of 7 event-timed steps).  hbm_frac
    counts the bytes the row's kernel has to move (for a fused kernel fewer than the reference sequence it
    replaces: Loihi forward + delayShift 16 + 8 B, Loihi backward 12 + 8 B)."""
    from slayerpytorch_amd import slayerCuda, slayerLoihiCuda
    from slayerpytorch_amd.slayer import alphaKernel
    from slayerpytorch_amd.slayerLoihi import loihiPspKernel

    def timed(fn, burst=1, args=None):
        """Median over 7 event-timed passes of the time per call; a pass is `burst` calls back to back (kernel rows:
        8, so that the few microseconds an event pair costs do not count as kernel time), each with its own
        argument from `args` when the op works in place."""
        ts = []
        for i in range(10):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            if args is not None:
                args[1]()                      # restore the in-place operands (untimed)
                torch.cuda.synchronize()
            a.record()
            for k in range(burst):
                fn(args[0][k]) if args is not None else fn()
            b.record()
            torch.cuda.synchronize()
            if i >= 3:
                ts.append(a.elapsed_time(b) * 1e-3 / burst)
        return float(np.median(ts))

    K = 8

    def row(name, ab, numel, seconds, shape, moved=None):
        """``ab``: algorithmic bytes per neuron-timestep of the reference sequence the row stands for.  A fused
        kernel (``moved`` given) moves fewer: its roofline fraction ``hbm_frac`` counts the bytes it moves, and the
        traffic the separate calls would have needed, over the same time, is kept under a name that cannot be read
        as a roofline fraction (it exceeds 1 where fusion saves traffic)."""
        r = {"op": name, "shape": list(shape), "us": seconds * 1e6, "neuron_timesteps_per_s": numel / seconds}
        if moved is None:
            r["hbm_frac"] = ab * numel / seconds / 1e9 / HBM_PEAK_GBS
        else:
            r["bytes_per_element_moved"] = moved
            r["hbm_frac"] = r["hbm_frac_of_bytes_moved"] = moved * numel / seconds / 1e9 / HBM_PEAK_GBS
            r["bytes_per_element_of_the_separate_calls"] = ab
            r["separate_calls_traffic_over_this_time_vs_hbm_peak"] = ab * numel / seconds / 1e9 / HBM_PEAK_GBS
        return r

    def cold(r, ab, src, fn):
        """Adds to row ``r`` the time of ``fn(input)`` when the input is not in the 256 MB last-level cache: a different
        copy of ``src`` per launch, more than 512 MB of copies in turn.  The row's own figure re-reads one input, which
        kernels that load with the default cache policy find in that cache when the tensor fits it."""
        copies = [src.clone() for _ in range(max(2, -(-(640 << 20) // (src.numel() * 4))))]
        burst = [copies[i % len(copies)] for i in range(K)]
        t = timed(lambda x: fn(x), K, (burst, lambda: None))
        r["us_with_input_not_in_cache"] = t * 1e6
        r["hbm_frac_with_input_not_in_cache"] = ab * src.numel() / t / 1e9 / HBM_PEAK_GBS
        return r

    def potentials(shape, srm_k, ref_k, tau_sr, rate_target):
        """A membrane potential of the kind real layers see: the PSP signal of Bernoulli(0.05) spikes - smooth, above
        the threshold for runs of samples - scaled so that about ``rate_target`` of the samples fire."""
        gp = torch.Generator(device="cpu").manual_seed(11)
        a = slayerCuda.pspAlpha((torch.rand(shape, generator=gp) < 0.05).float().to(device), srm_k, tau_sr, 1.0, 1.0, True)
        lo, hi = 0.05, 2000.0
        for _ in range(16):
            gain = (lo * hi) ** 0.5
            rate = float(slayerCuda.getSpikes(a * gain, ref_k, 10.0, 1.0).mean())
            lo, hi = (gain, hi) if rate < rate_target else (lo, gain)
        u = (a * gain).contiguous()
        return u, rate, float((u >= 10.0).float().mean())

    def spike_on_potentials(name, shape, srm_k, ref_k, tau_sr, rate_target):
        u_real, rate, above = potentials(shape, srm_k, ref_k, tau_sr, rate_target)
        pool = [u_real.clone() for _ in range(K)]
        restore = lambda: [p.copy_(u_real) for p in pool]
        r = row(name, 12, u_real.numel(), timed(lambda u: slayerCuda.getSpikes(u, ref_k, 10.0, 1.0), K, (pool, restore)), shape)
        r["spike_rate"], r["samples_at_or_above_theta_before_the_walk"] = round(rate, 4), round(above, 4)
        return r

    out = []
    g = torch.Generator(device="cpu").manual_seed(2)
    # delay stress config: (64, 256, 1, 1, 2000), delays U[0, 62], 8-tap SRM kernel
    shape = (64, 256, 1, 1, 2000)
    x = (torch.rand(shape, generator=g) < 0.005).float().to(device)
    grad = torch.randn(shape, generator=g).to(device)
    lut = (torch.rand((256, 1, 1), generator=g) * 62).to(device)
    srm8 = torch.tensor(alphaKernel(1.0, 1.0, 2000), dtype=torch.float32, device=device)
    ref = torch.tensor(alphaKernel(1.0, 1.0, 2000, mult=-20.0), dtype=torch.float32, device=device)
    u0 = (torch.randn(shape, generator=g) * 5).to(device)
    ub = u0.clone()
    n = x.numel()
    y = slayerCuda.shift(x, lut, 1.0)
    out.append(row("shift_per_neuron_table", 8, n, timed(lambda: slayerCuda.shift(x, lut, 1.0), K), shape))
    out.append(row("delay_gradient", 8, n, timed(lambda: slayerCuda.delayGrad(y, grad, 1.0), K), shape))
    out.append(row("psp_conv_8tap", 8, n, timed(lambda: slayerCuda.conv(x, srm8, 1.0), K), shape))
    out.append(row("psp_corr_8tap", 8, n, timed(lambda: slayerCuda.corr(grad, srm8, 1.0), K), shape))
    pool = [u0.clone() for _ in range(K)]
    restore = lambda: [p.copy_(u0) for p in pool]
    out.append(row("spike_T2000", 12, n, timed(lambda u: slayerCuda.getSpikes(u, ref, 10.0, 1.0), K, (pool, restore)), shape))
    out.append(row("spike_T2000_then_per_neuron_delay_fused", 20, n,
                   timed(lambda u: slayerCuda.getSpikesDelayed(u, ref, 10.0, 1.0, lut, 1.0), K, (pool, restore)), shape, moved=12))
    del x, grad, u0, ub, y, pool
    # the 77-tap alpha kernel on these long rows: as a recursion carried from piece to piece, and as sums over the taps
    srm77 = torch.tensor(alphaKernel(10.0, 1.0, 2000), dtype=torch.float32, device=device)
    xg = torch.randn(shape, generator=g).to(device)
    for nm, src in (("spikes", (torch.rand(shape, generator=g) < 0.02).float().to(device)), ("dense", xg)):
        for causal in (True, False):
            r = row("psp_%s77_T2000_as_recursion_%s_input" % ("conv" if causal else "corr", nm), 8, n,
                    timed(lambda: slayerCuda.pspAlpha(src, srm77, 10.0, 1.0, 1.0, causal), K), shape)
            taps = timed(lambda: (slayerCuda.conv if causal else slayerCuda.corr)(src, srm77, 1.0), K)
            r["us_as_sums_over_the_taps"], r["hbm_frac_as_sums_over_the_taps"] = taps * 1e6, 8 * n / taps / 1e9 / HBM_PEAK_GBS
            if nm == "dense":
                cold(r, 8, src, lambda x: slayerCuda.pspAlpha(x, srm77, 10.0, 1.0, 1.0, causal))
            out.append(r)
    del xg, src
    # the spike kernel's time depends on its input: the rows above (and the headline) feed independent normal samples
    # (2.3 % isolated samples at or above the threshold); real potentials are smooth and stay above it for runs of samples
    out.append(spike_on_potentials("spike_T2000_on_psp_shaped_potential_firing_4_percent", shape, srm8, ref, 1.0, 0.04))
    srm77, ref11 = (torch.tensor(alphaKernel(tau, 1.0, 300, mult=m), dtype=torch.float32, device=device) for tau, m in ((10.0, 1.0), (1.0, -20.0)))
    for target in (0.04, 0.30):
        out.append(spike_on_potentials("spike_on_psp_shaped_potential_firing_%d_percent" % round(100 * target),
                                       (12, 16, 32, 32, 300), srm77, ref11, 10.0, target))
    # the 77-tap PSP filter over the density of its input, as the sum over the taps (slayerCuda.conv: spike trains
    # take the event-driven path tile by tile, denser tiles the matrix cores) and as the recursion that the layers
    # run for their own alpha kernel
    shape = SHAPE
    srm77 = torch.tensor(alphaKernel(10.0, 1.0, 300), dtype=torch.float32, device=device)
    for p in (0.02, 0.05, 0.10, 0.40, None):
        xin = (torch.randn(shape, generator=g) if p is None else (torch.rand(shape, generator=g) < p).float()).to(device)
        r = row("psp_conv77_input_density_%s" % ("dense" if p is None else "%.2f" % p), 8, xin.numel(),
                timed(lambda: slayerCuda.conv(xin, srm77, 1.0), K), shape)
        rec = timed(lambda: slayerCuda.pspAlpha(xin, srm77, 10.0, 1.0, 1.0, True), K)
        r["us_as_recursion"] = rec * 1e6
        r["hbm_frac_as_recursion"] = 8 * xin.numel() / rec / 1e9 / HBM_PEAK_GBS
        out.append(r)
        del xin
    # MLP ordering spike(psp(fc(x))): dense input to the 77-tap PSP filter, then the spike function
    shape = SHAPE
    a = (torch.randn(shape, generator=g) * 2).to(device)
    ref11 = torch.tensor(alphaKernel(1.0, 1.0, 300, mult=-20.0), dtype=torch.float32, device=device)
    out.append(row("psp77_then_spike_fused", 20, a.numel(), timed(lambda: slayerCuda.pspSpike(a, srm77, ref11, 10.0, 1.0), K),
                   shape, moved=12))
    out.append(row("psp77_then_spike_two_kernels", 20, a.numel(),
                   timed(lambda: slayerCuda.getSpikes(slayerCuda.conv(a, srm77, 1.0), ref11, 10.0, 1.0), K), shape))
    # ... as the layers run it for their alpha kernel: the recursion over time, then the spike kernel
    out.append(row("psp77_as_recursion_then_spike_two_kernels", 20, a.numel(),
                   timed(lambda: slayerCuda.getSpikes(slayerCuda.pspAlpha(a, srm77, 10.0, 1.0, 1.0, True), ref11, 10.0, 1.0), K), shape))
    out.append(row("psp77_as_recursion_dense_input", 8, a.numel(), timed(lambda: slayerCuda.pspAlpha(a, srm77, 10.0, 1.0, 1.0, True), K), shape))
    gs = torch.randn(shape, generator=g).to(device)
    out.append(row("spike_pdf_then_corr77_fused", 20, a.numel(),
                   timed(lambda: slayerCuda.spikeBackwardCorr(gs, a, srm77, 10.0, 10.0, 1.0, 1.0), K), shape, moved=12))
    # ... for the layers' alpha kernel: the surrogate gradient on the way in, the correlation as a recursion
    out.append(row("spike_pdf_then_corr77_as_recursion_fused", 20, a.numel(),
                   timed(lambda: slayerCuda.spikeBackwardPspAlpha(gs, a, srm77, 10.0, 1.0, 10.0, 10.0, 1.0, 1.0), K), shape, moved=12))
    del a, gs
    # NMNIST-shaped MLP end to end (dense layers are library GEMMs): forward, spike-time loss, backward
    out.append(mlp_row(device, timed))
    # NMNIST-shaped CNN end to end (synapses by the per-timestep synapse kernels)
    out.append(cnn_row(device, timed))
    out.append(delay_mlp_row(device, timed))
    out.extend(synapse_rows(device, timed))
    out.append(event_row(device, timed, cpu_leg))
    out.append(loihi_cnn_row(device, timed))
    # Loihi config: largest tensor (8, 16, 32, 32, 300)
    shape = (8, 16, 32, 32, 300)
    w = (2 * torch.randint(-128, 128, shape, generator=g) * (torch.rand(shape, generator=g) < 0.05)).float().to(device)
    gl = torch.randn(shape, generator=g).to(device)
    psp = torch.tensor(loihiPspKernel(1024, 128, 0), dtype=torch.float32, device=device)
    n = w.numel()
    s, v, u = slayerLoihiCuda.getSpikes(w, 0, 5120, 1024, 128, 1)
    out.append(cold(row("loihi_forward", 16, n, timed(lambda: slayerLoihiCuda.getSpikes(w, 0, 5120, 1024, 128, 1), K), shape),
                    16, w, lambda x: slayerLoihiCuda.getSpikes(x, 0, 5120, 1024, 128, 1)))
    out.append(row("loihi_forward_spike_and_voltage_delay1_fused", 24, n,
                   timed(lambda: slayerLoihiCuda.getSpikesDelayed(w, 0, 5120, 1024, 128, 1, 1, voltage=True, current=False), K),
                   shape, moved=12))
    out.append(row("loihi_forward_spike_only_delay1_fused", 24, n,
                   timed(lambda: slayerLoihiCuda.getSpikesDelayed(w, 0, 5120, 1024, 128, 1, 1, voltage=False, current=False), K),
                   shape, moved=8))
    cold(out[-1], 8, w, lambda x: slayerLoihiCuda.getSpikesDelayed(x, 0, 5120, 1024, 128, 1, 1, voltage=False, current=False))
    out.append(row("loihi_backward_pdf_plus_corr110", 20, n,
                   timed(lambda: slayerCuda.spikeBackwardCorr(gl, v, psp, 5120.0, 5120.0, 1 / 195.0, 1.0), K),
                   shape, moved=12))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true",
                    help="skip the CPU leg (oracle baseline timing and the spike flip rate against it)")
    ap.add_argument("--chain-only", action="store_true",
                    help="only the headline chain (for profiler runs): no per-kernel pass, flip rate, "
                         "other rows or CPU baseline")
    ap.add_argument("--cnn-only", action="store_true",
                    help="only the NMNIST CNN training step of the other rows (for profiler runs); prints that row")
    ap.add_argument("--mlp-only", action="store_true",
                    help="only the NMNIST MLP training step of the other rows (for profiler runs); prints that row")
    ap.add_argument("--delay-only", action="store_true",
                    help="only the long-sequence delay network's training step (for profiler runs); prints that row")
    ap.add_argument("--loihi-only", action="store_true",
                    help="only the Loihi gesture network's inference and training steps (for profiler runs); prints that row")
    ap.add_argument("--synapse-only", action="store_true",
                    help="only the per-layer synapse kernel rows (for profiler runs); prints those rows")
    ap.add_argument("--dense-conv", action="store_true",
                    help="also launch, in every warm-up step, the kernels that sum over the 77 taps: conv on a dense input "
                         "(the gradient tensor: matrix cores), conv on the spike tensor (event-driven) and corr on the "
                         "gradient tensor (matrix cores) (for profiler runs)")
    ap.add_argument("--tap-kernels-chain", action="store_true",
                    help="psp and its gradient in the chain as sums over the 77 taps (slayerCuda.conv / corr) instead "
                         "of the recursion that the layers use for their alpha kernel")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also launch one plain copy of known size (a zero-delay shift of half the tensor: "
                         "%d bytes read, as many written) to scale hardware counters by" % (4 * 6 * 16 * 34 * 34 * 300))
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: every kernel on this path treats neuron rows independently, "
                 "so N GPUs is N independent copies of this run; use --gpus 1")
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")

    from slayerpytorch_amd import slayerCuda
    from slayerpytorch_amd.slayer import alphaKernel

    device = torch.device("cuda:0")
    torch.cuda.set_device(device)
    if args.cnn_only or args.mlp_only or args.synapse_only or args.delay_only or args.loihi_only:
        def wall(fn):
            ts = []
            for _ in range(args.warmup + args.steps):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                fn()
                torch.cuda.synchronize()
                ts.append(time.perf_counter() - t0)
            return float(np.median(ts[args.warmup:]))
        if args.cnn_only:
            print(json.dumps(cnn_row(device, wall)))
        elif args.mlp_only:
            print(json.dumps(mlp_row(device, wall)))
        elif args.delay_only:
            print(json.dumps(delay_mlp_row(device, wall)))
        elif args.loihi_only:
            print(json.dumps(loihi_cnn_row(device, wall)))
        else:
            print(json.dumps({"synapse_rows": synapse_rows(device, wall)}))
        return
    params = neuron_params()
    srm = np.array(alphaKernel(params["tauSr"], 1.0, SHAPE[-1]), dtype=np.float32)
    ref = np.array(alphaKernel(params["tauRef"], 1.0, SHAPE[-1], mult=-params["scaleRef"] * params["theta"]),
                   dtype=np.float32)
    srm_t, ref_t = torch.from_numpy(srm).to(device), torch.from_numpy(ref).to(device)
    theta, tau, scale = params["theta"], params["tauRho"] * params["theta"], params["scaleRho"]

    spikes, u0, grad = make_inputs(SHAPE, device)
    numel = spikes.numel()
    # psp and its gradient as spikeLayer.psp runs them: the layer's SRM kernel is an alpha kernel, which it filters
    # as a recursion over time (same results as the sum over the 77 taps to rounding); --tap-kernels-chain times
    # the chain with the sums instead, and the full run reports both
    if args.tap_kernels_chain:
        psp_fwd = lambda x: slayerCuda.conv(x, srm_t, 1.0)
        psp_bwd = lambda g: slayerCuda.corr(g, srm_t, 1.0)
        KERNEL_OF["psp_conv"] = "slayer::fir_tiled_kernel<true, true, 16, false, 6> (conv as a sum over the taps; spike trains: event-driven path)"
        KERNEL_OF["psp_corr"] = "slayer::fir_mfma_kernel<6, 20, true, false> (corr as a sum over the taps, matrix cores)"
    else:
        psp_fwd = lambda x: slayerCuda.pspAlpha(x, srm_t, params["tauSr"], 1.0, 1.0, True)
        psp_bwd = lambda g: slayerCuda.pspAlpha(g, srm_t, params["tauSr"], 1.0, 1.0, False)
    names = list(AB)
    probe = 0 if args.chain_only else max(args.steps, 1)   # untimed steps with an event pair around every launch
    pool = [u0.clone() for _ in range(args.warmup + probe + args.steps)]   # spike() consumes one copy per step

    def event_pair():
        return torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)

    def step(u, ev=None):
        """ev: {op index: (start, stop)} - the launches to bracket with HIP events (torch records
        them on the current stream, which is the stream the kernels are launched on)."""
        def run(k, fn):
            if ev is not None and k in ev:
                ev[k][0].record()
            out = fn()
            if ev is not None and k in ev:
                ev[k][1].record()
            return out

        run(0, lambda: psp_fwd(spikes))
        s = run(1, lambda: slayerCuda.getSpikes(u, ref_t, theta, 1.0))
        run(2, lambda: slayerCuda.shift(s, 1.0, 1.0))
        gd = run(3, lambda: slayerCuda.shift(grad, 1.0, 1.0, sign=-1.0))
        gs = run(4, lambda: slayerCuda.spikeBackward(gd, u, theta, tau, scale))
        run(5, lambda: psp_bwd(gs))

    for i in range(args.warmup):
        step(pool[i])
        if args.dense_conv:
            for _ in range(3):
                slayerCuda.conv(grad, srm_t, 1.0)
                slayerCuda.conv(spikes, srm_t, 1.0)
                slayerCuda.corr(grad, srm_t, 1.0)
    if args.copy_calibration:
        slayerCuda.shift(grad[:6], 0.0, 1.0)
    torch.cuda.synchronize()

    # Per-kernel pass (untimed): every launch bracketed.  The event records themselves cost a few
    # microseconds per launch, so the timed region below brackets the dominant kernel only.
    per_kernel_ms = None
    dominant = "spike"
    if probe:
        evs = [{k: event_pair() for k in range(len(names))} for _ in range(probe)]
        for i in range(probe):
            step(pool[args.warmup + i], evs[i])
        torch.cuda.synchronize()
        per_kernel_ms = {n: float(np.mean([evs[i][k][0].elapsed_time(evs[i][k][1]) for i in range(probe)]))
                         for k, n in enumerate(names)}
        dominant = max(per_kernel_ms, key=per_kernel_ms.get)
    kd = names.index(dominant)

    evs = [{kd: event_pair()} for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(pool[args.warmup + probe + i], evs[i])
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    ms_per_step = elapsed / args.steps * 1e3
    dominant_ms = float(np.mean([evs[i][kd][0].elapsed_time(evs[i][kd][1]) for i in range(args.steps)]))
    achieved = AB[dominant] * numel / (dominant_ms * 1e-3) / 1e9
    chain_gbs = sum(AB.values()) * numel / (elapsed / args.steps) / 1e9

    result = {
        "metric": "neuron-timesteps/s spike+psp+shift fwd/bwd at 1 MI355X; % HBM peak GB/s",
        "value": numel / (elapsed / args.steps),
        "unit": "neuron-timesteps/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "NMNIST-CNN-shaped activation tensor (12,16,34,34,300): psp conv (77-tap alpha kernel) + "
                               "spike (11-tap refractory) + shift fwd, shift + spike pdf + psp corr bwd",
                   "elements": numel, "algorithmic_bytes_per_element": sum(AB.values())},
        "roofline": {"bound": "hbm", "kernel": KERNEL_OF[dominant], "op": dominant, "achieved": achieved,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "launch_ms": dominant_ms,
                     "traffic": measured_traffic(dominant)[0], "traffic_source": measured_traffic(dominant)[1]},
        # the whole step (six launches and the gaps between them) against the HBM peak
        "chain_hbm_frac": chain_gbs / HBM_PEAK_GBS,
    }
    # summed over their 77 taps the filters sit at the FP32 ridge: then also as a fraction of the FP32 peak
    result["roofline"]["fp32_frac_if_fir"] = (2.0 * SRM_TAPS * numel / (dominant_ms * 1e-3) / 1e12 / FP32_PEAK_TFLOPS
                                              if args.tap_kernels_chain and dominant in ("psp_conv", "psp_corr") else None)
    if per_kernel_ms is not None:
        result["per_kernel_ms"] = per_kernel_ms
        result["per_kernel_hbm_frac"] = {n: AB[n] * numel / (per_kernel_ms[n] * 1e-3) / 1e9 / HBM_PEAK_GBS
                                         for n in names}
        result["per_kernel_pass"] = "%d untimed steps before the timed region, an event pair around every launch" % probe
    del pool
    if not args.chain_only:
        # The same step with the shift fused into the spike kernel (forward) and into the surrogate
        # gradient (backward): four launches, 40 instead of 56 bytes per element, same results.
        pool = [u0.clone() for _ in range(args.warmup + args.steps + 2)]

        def fused_step(u):
            psp_fwd(spikes)
            slayerCuda.getSpikesDelayed(u, ref_t, theta, 1.0, 1.0, 1.0)
            gs = slayerCuda.spikeBackwardDelayed(grad, u, theta, tau, scale, 1.0, 1.0)
            psp_bwd(gs)

        for i in range(args.warmup):
            fused_step(pool[i])
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            fused_step(pool[args.warmup + i])
        torch.cuda.synchronize()
        fused = (time.perf_counter() - t0) / args.steps
        ua, ub = pool[-1], pool[-2]
        same = bool(torch.equal(slayerCuda.getSpikesDelayed(ua, ref_t, theta, 1.0, 1.0, 1.0),
                                slayerCuda.shift(slayerCuda.getSpikes(ub, ref_t, theta, 1.0), 1.0, 1.0))
                    and torch.equal(slayerCuda.spikeBackwardDelayed(grad, ua, theta, tau, scale, 1.0, 1.0),
                                    slayerCuda.spikeBackward(slayerCuda.shift(grad, 1.0, 1.0, sign=-1.0), ub, theta, tau,
                                                             scale)))
        result["fused_shift_chain"] = {
            "launches": "psp conv, spike+shift | shift+spike pdf, psp corr", "ms_per_step": fused * 1e3,
            "value": numel / fused, "unit": "neuron-timesteps/s", "algorithmic_bytes_per_element": 40,
            "hbm_frac": 40 * numel / fused / 1e9 / HBM_PEAK_GBS, "identical_to_unfused_results": same}
        del pool
        if not args.tap_kernels_chain:
            # the chain's two filters as sums over the taps (what slayerCuda.conv / corr run for any filter)
            K = max(args.steps, 5)
            def timed_us(fn):
                for _ in range(3):
                    fn()
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(K):
                    fn()
                torch.cuda.synchronize()
                return (time.perf_counter() - t0) / K * 1e6
            gs = slayerCuda.spikeBackward(grad, u0, theta, tau, scale)
            tc, tr = timed_us(lambda: slayerCuda.conv(spikes, srm_t, 1.0)), timed_us(lambda: slayerCuda.corr(gs, srm_t, 1.0))
            ya, yt = psp_fwd(spikes), slayerCuda.conv(spikes, srm_t, 1.0)
            za, zt = psp_bwd(gs), slayerCuda.corr(gs, srm_t, 1.0)
            result["psp_as_sums_over_the_taps"] = {
                "psp_conv_us": tc, "psp_corr_us": tr,
                "psp_conv_hbm_frac": 8 * numel / (tc * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "psp_corr_hbm_frac": 8 * numel / (tr * 1e-6) / 1e9 / HBM_PEAK_GBS,
                "ms_per_step_with_them": ms_per_step + (tc + tr) * 1e-3 - (per_kernel_ms["psp_conv"] + per_kernel_ms["psp_corr"]),
                "recursion_vs_sums_max_rel_diff": {"conv": float((ya - yt).abs().max() / yt.abs().max()),
                                                    "corr": float((za - zt).abs().max() / zt.abs().max())}}
            del gs, ya, yt, za, zt
        result["measured_copy_ceiling"] = copy_ceiling(grad)
        result["other_rows"] = other_rows(device, cpu_leg=not args.no_cpu_baseline)
        if not args.no_cpu_baseline:
            # the CPU leg: the oracle as the timed baseline and as the checker of the flip rate
            result["cpu_baseline"] = cpu_baseline(SHAPE, srm, ref, params)
            result["cpu_baseline"]["cpu_model"] = cpu_model()
            result["cpu_baseline"]["host_cpu_count"] = os.cpu_count()
            result["cpu_baseline_plumbing_case"] = cpu_plumbing_baseline(srm, ref, params)
            flips, rate = flip_rate(device, srm_t, ref_t, params)
            result["spike_flip_rate"] = flips
            result["spike_rate"] = rate
            lflips, lrate = layer_flip_rate(device, srm_t, ref_t, params)
            result["cnn_layer_spike_flip_rate"] = lflips
            result["cnn_layer_spike_rate"] = lrate
    print(json.dumps(result))


if __name__ == "__main__":
    main()

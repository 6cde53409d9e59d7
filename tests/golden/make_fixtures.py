"""Regenerates the golden fixtures under tests/golden/ from the data files that the
reference keeps for its own tests.

Run once, in the development container, where the reference tree is mounted:

    python tests/golden/make_fixtures.py [/root/reference]

It only *reads data files* (text tables of spikes, weights, kernels, recorded voltages); no
reference code is imported or executed.  The resulting ``.npz`` archives are committed, so the
tests never need the reference tree.  Every array keeps the layout of the file it came from;
dense 0/1 rasters are stored as event lists to keep the archives small.
"""
import os
import sys

import numpy as np

REF = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
TF = os.path.join(REF, "test", "test_files")
OUT = os.path.dirname(os.path.abspath(__file__))


def txt(path, **kw):
    return np.loadtxt(os.path.join(TF, path), **kw)


def csv(path):
    return np.loadtxt(os.path.join(TF, path), delimiter=",", ndmin=2)


def events(raster):
    """(row, column, value) triplets of the non-zero entries of a 2-D raster."""
    r, c = np.nonzero(raster)
    return np.stack([r, c], 1).astype(np.int32), raster[r, c].astype(np.float32)


def save(name, **arrays):
    path = os.path.join(OUT, name)
    np.savez_compressed(path, **arrays)
    print("%-28s %8.1f KiB" % (name, os.path.getsize(path) / 1024))


# --- test/test_files/snnData: MATLAB-SLAYER ground truth for the 250-25-1 network, Ts=0.1 ----
save(
    "snn_250_25_1.npz",
    h_sr=txt("snnData/h_sr.txt").astype(np.float32),              # (77, 2): time, SRM kernel
    h_ref=txt("snnData/h_ref.txt").astype(np.float32),            # (110, 2): time, refractory kernel
    spikeFuncHid=txt("snnData/spikeFuncHid.txt").astype(np.float32),      # (501, 3): u, u+ref, spike
    spikeFuncHid04=txt("snnData/spikeFuncHid04.txt").astype(np.float32),
    spikeFuncOut=txt("snnData/spikeFuncOut.txt").astype(np.float32),
    spikeIn=txt("snnData/spikeIn.txt").astype(np.float32),        # AER (time ms, 1-based neuron)
    spikeHid=txt("snnData/spikeHid.txt").astype(np.float32),
    spikeOut=txt("snnData/spikeOut.txt").astype(np.float32),
    w1learned=txt("snnData/w1learned.txt").astype(np.float32),    # (25, 250)
    w2learned=txt("snnData/w2learned.txt", ndmin=2).astype(np.float32),   # (1, 25)
    w1Initial=txt("snnData/w1Initial.txt").astype(np.float32),
    w2Initial=txt("snnData/w2Initial.txt", ndmin=2).astype(np.float32),
    gradW1Initial=txt("snnData/gradW1Initial.txt").astype(np.float32),
    gradW2Initial=txt("snnData/gradW2Initial.txt", ndmin=2).astype(np.float32),
)

# --- test/test_files/Loihi/LoihiData: recordings from a Loihi chip ------------------------------
with open(os.path.join(TF, "Loihi/LoihiData/LoihiVth05.txt")) as f:
    vth_rows = [np.array([int(x) for x in line.replace(",", " ").split()], dtype=np.int32)
                for line in f if line.strip()]
save(
    "loihi_chip.npz",
    hiddenSpikes=txt("Loihi/LoihiData/loihiHiddenSpikes.txt").astype(np.int32),   # (neuron, time)
    outputSpikes=txt("Loihi/LoihiData/loihiOutputSpikes.txt", ndmin=2).astype(np.int32),
    inputSpikes=txt("Loihi/LoihiData/loihiInputSpikes.txt").astype(np.int32),
    hiddenVoltage24=txt("Loihi/LoihiData/loihiHiddenVoltage24.txt").astype(np.int32),
    hiddenVoltage23=txt("Loihi/LoihiData/loihiHiddenVoltage23.txt").astype(np.int32),
    outputVoltage=txt("Loihi/LoihiData/loihiOutputVoltage.txt").astype(np.int32),
    impulseVoltage=vth_rows[1],       # second row: voltage trace after one weight-2 input spike
)

# --- test/test_files/torch_validate: legacy C++/MATLAB traces (Ts=0.1, 250-25-1) ---------------
s1_ev, s1_val = events(csv("torch_validate/forward_prop/s1.csv"))
save(
    "torch_validate.npz",
    refractory_kernel=csv("torch_validate/refractory_kernel.csv")[0].astype(np.float32),
    s1_shape=np.array([250, 501], dtype=np.int32), s1_events=s1_ev, s1_values=s1_val,
    a1=csv("torch_validate/forward_prop/a1.csv").astype(np.float32),
    W12=csv("torch_validate/forward_prop/W12.csv").astype(np.float32),
    W23=csv("torch_validate/forward_prop/W23.csv").astype(np.float32),
    u2=csv("torch_validate/forward_prop/u2.csv").astype(np.float32),
    s2=csv("torch_validate/forward_prop/s2.csv").astype(np.float32),
    u3=csv("torch_validate/forward_prop/u3.csv").astype(np.float32),
    s3=csv("torch_validate/forward_prop/s3.csv").astype(np.float32),
    a3=csv("torch_validate/forward_prop/a3.csv").astype(np.float32),
    des_s=csv("torch_validate/back_prop/des_s.csv").astype(np.float32),
    des_a=csv("torch_validate/back_prop/des_a.csv").astype(np.float32),
    e3=csv("torch_validate/back_prop/e3.csv").astype(np.float32),
    rho3=csv("torch_validate/back_prop/rho3.csv").astype(np.float32),
    Wgrad1=csv("torch_validate/back_prop/Wgrad1.csv").astype(np.float32),
    Wgrad2=csv("torch_validate/back_prop/Wgrad2.csv").astype(np.float32),
)

# --- input_validate -> torch_validate spike response of one NMNIST sample (2312 x 350) ---------
ROWS = slice(0, None, 1)
b1 = csv("input_validate/1_binned_spikes.csv")[ROWS]
b2 = csv("input_validate/1_binned_spikes_ts2.csv")[ROWS]
ev1, val1 = events(b1)
ev2, val2 = events(b2)
save(
    "nmnist_response.npz",
    row_step=np.array(1, dtype=np.int32),
    binned_shape=np.array(b1.shape, dtype=np.int32), binned_events=ev1, binned_values=val1,
    response=csv("torch_validate/1_spike_response_signal.csv")[ROWS].astype(np.float32),
    binned_ts2_shape=np.array(b2.shape, dtype=np.int32), binned_ts2_events=ev2, binned_ts2_values=val2,
    response_ts2=csv("torch_validate/1_spike_response_signal_ts2.csv")[ROWS].astype(np.float32),
)

# --- spike event files: the reference's own sample in three forms -------------------------------
# NMNISTsmall/1.bs2 (packed events) <-> input_validate/1_raw_spikes.csv (x, y, p, t in us, 1-based
# x/y/p) <-> the binned rasters already read above (b1: 1 ms bins, b2: 2 ms bins; both binned by
# truncation).  Plus one 1-D file and the head of one 3-D file for the other two byte layouts.
def raw_bytes(path, limit=None):
    with open(os.path.join(TF, path), "rb") as f:
        data = f.read() if limit is None else f.read(limit)
    return np.frombuffer(data, dtype=np.uint8).copy()


save(
    "spike_events.npz",
    nmnist_bs2=raw_bytes("NMNISTsmall/1.bs2"),
    nmnist_raw=np.loadtxt(os.path.join(TF, "input_validate/1_raw_spikes.csv"), delimiter=",", skiprows=1).astype(np.int32),
    ntidigits_bs1=raw_bytes("binarySpikeTestFiles/NTIDIGITS_1.bs1"),
    sample_bs3=raw_bytes("binarySpikeTestFiles/1.bs3", 7 * 3000),
)

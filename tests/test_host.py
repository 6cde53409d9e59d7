"""Host-side checks that need no GPU: the C-ABI library loads and exports every symbol the
header declares, and the Python modules reject bad arguments before anything is launched, with
the error behaviour of the reference bindings (src/cuda/slayerKernels.cu:7-10, 35, 102;
src/cuda/slayerLoihiKernels.cu:12-19)."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from slayerpytorch_amd import _lib, slayerCuda, slayerLoihiCuda
import slayerpytorch_amd as snn

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "slayer_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(slayer_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 13 and "slayer_conv_f32" in names and "slayer_loihi_get_spikes_f32" in names
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in names:
        assert hasattr(lib, name), "libslayer_hip.so does not export %s" % name
    assert sorted(_lib.SIGNATURES) == names, "python binding table and header disagree"


def test_abi_version_and_status_strings():
    lib = _lib.load()
    assert lib.slayer_hip_abi_version() == _lib.ABI_VERSION == 1
    assert lib.slayer_status_string(0) == b"ok"
    assert lib.slayer_status_string(1) == b"invalid argument"
    assert lib.slayer_status_string(77) == b"unknown status"
    with pytest.raises(_lib.SlayerHipError, match="invalid argument"):
        _lib.check(1, "slayer_conv_f32")


def test_argument_validation_in_the_c_abi_without_launch():
    lib = _lib.load()
    # empty tensors are a successful no-op, whatever the pointers
    assert lib.slayer_conv_f32(None, None, None, 0, 10, 3, 1.0, None) == 0
    assert lib.slayer_get_spikes_f32(None, None, None, 5, 0, 3, 1.0, 1.0, None) == 0
    # null pointers with work to do, negative sizes, refDelay 0, bad sign
    assert lib.slayer_conv_f32(None, None, None, 4, 10, 3, 1.0, None) == 1
    assert lib.slayer_corr_f32(None, None, None, -1, 10, 3, 1.0, None) == 1
    assert lib.slayer_shift_f32(None, None, 1.0, 4, 10, 1.0, None) == 1
    assert lib.slayer_shift_lut_f32(None, None, None, 3, 2, 4, 10, 1.0, 1.0, None) == 1     # lutSize != nPerBatch
    assert lib.slayer_shift_lut_f32(None, None, None, 4, 0, 4, 10, 1.0, 0.5, None) == 1     # sign must be +-1
    assert lib.slayer_loihi_get_spikes_f32(None, None, None, None, 0, 0, 0, 64, 0, 0, 0, None) == 1   # refDelay 0
    assert lib.slayer_loihi_get_spikes_f32(None, None, None, None, 0, 0, 26, 64, 0, 0, 1, None) == 1  # 1 << 32
    assert lib.slayer_spike_bwd_f32(None, None, None, 1.0, 0.0, 1.0, 4, None) == 1
    assert lib.slayer_delay_grad_workspace_bytes(64, 256, 2000) == 64 * 256 * 4
    assert lib.slayer_delay_grad_workspace_bytes(0, 256, 2000) == 0


def test_cpu_tensors_are_rejected_like_the_reference():
    x = torch.zeros(1, 2, 1, 1, 10)
    f = torch.ones(3)
    for call in (lambda: slayerCuda.conv(x, f, 1.0), lambda: slayerCuda.corr(x, f, 1.0),
                 lambda: slayerCuda.shift(x, f, 1.0), lambda: slayerCuda.shift(x, 1.0),
                 lambda: slayerCuda.getSpikes(x, f, 1.0, 1.0),
                 lambda: slayerLoihiCuda.getSpikes(x, 0, 64, 0, 0, 1),
                 lambda: slayerLoihiCuda.getSpikesDelayed(x, 0, 64, 0, 0, 1, 1, voltage=False),
                 lambda: slayerCuda.pspSpike(x, f, f, 1.0, 1.0),
                 lambda: slayerCuda.spikeBackward(x, x, 1.0, 1.0, 1.0),
                 lambda: slayerCuda.spikeBackwardCorr(x, x, f, 1.0, 1.0, 1.0, 1.0),
                 lambda: slayerCuda.delayGrad(x, x, 1.0)):
        with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
            call()


def test_non_tensor_and_bad_scalar_arguments():
    f = torch.ones(3)
    with pytest.raises(TypeError):
        slayerCuda.conv([1.0, 2.0], f, 1.0)
    with pytest.raises(TypeError):
        slayerLoihiCuda.getSpikes(None, 0, 64, 0, 0, 1)


def test_loihi_integer_arguments_follow_unsigned_conversion():
    from slayerpytorch_amd.slayerLoihiCuda import _unsigned
    assert _unsigned(5, "x") == 5 and _unsigned(torch.tensor(7), "x") == 7
    import numpy as np
    assert _unsigned(np.int64(3), "x") == 3
    for bad in (-1, 1.5, "3", 1 << 32, torch.tensor(1.0)):
        with pytest.raises(TypeError):
            _unsigned(bad, "x")


def test_scalar_conversion_accepts_numbers_and_one_element_tensors():
    from slayerpytorch_amd.slayerCuda import _scalar
    import numpy as np
    assert _scalar(2, "Ts") == 2.0 and _scalar(torch.tensor(0.5), "Ts") == 0.5
    assert _scalar(np.float32(0.25), "Ts") == 0.25
    with pytest.raises(TypeError):
        _scalar(torch.ones(2), "Ts")
    with pytest.raises(TypeError):
        _scalar("1.0", "Ts")


def test_layer_objects_build_without_gpu():
    neuron = {"theta": 10, "tauSr": 10.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    layer = snn.layer(neuron, {"Ts": 1.0, "tSample": 300})
    assert layer.srmKernel.numel() == 77 and layer.refKernel.numel() == 11
    assert set(layer.state_dict()) == {"srmKernel", "refKernel"}        # buffers travel with the state dict
    assert layer.refKernel[1].item() == pytest.approx(-20.0)
    delay = layer.delay((4, 3, 2))
    assert delay.delay.shape == (4, 3, 2) and delay.delay.requires_grad
    assert layer.delay(5).delay.shape == (5, 1, 1)
    fc = layer.dense(12, 7)
    assert fc.weight.shape == (7, 12, 1, 1, 1)
    assert layer.dense((3, 4, 2), 5).weight.shape == (5, 2, 4, 3, 1)
    ld = {"type": "LOIHI", "vThMant": 80, "vDecay": 128, "iDecay": 1024, "refDelay": 1, "wgtExp": 0,
          "tauRho": 1, "scaleRho": 1}
    loihi = snn.loihi(ld, {"Ts": 1, "tSample": 300})
    assert ld["theta"] == 5120 and loihi.maxPspKernel == 195.0 and ld["scaleRho"] == pytest.approx(1 / 195.0)
    w = loihi.dense(8, 4)
    q = w.preHookFx(w.weight)
    assert torch.all(q == torch.round(q / 2) * 2)                        # weights quantised in steps of 2


def test_dense_layer_as_matrix_product_equals_the_3d_convolution():
    # the reference's dense layer is a conv3d whose kernel spans the whole (H, W) extent; the same
    # numbers from one matrix product per batch item (time stays innermost)
    import torch.nn.functional as F
    neuron = {"theta": 10, "tauSr": 1.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    layer = snn.layer(neuron, {"Ts": 1.0, "tSample": 50})
    torch.manual_seed(0)
    for inF, shape in (((3, 4, 2), (2, 2, 4, 3, 17)), (12, (3, 12, 1, 1, 9)), ((5, 2), (1, 1, 2, 5, 4))):
        fc = layer.dense(inF, 6)
        x = torch.randn(shape, requires_grad=True)
        y = fc(x)
        ref = F.conv3d(x, fc.weight)
        assert y.shape == ref.shape == (shape[0], 6, 1, 1, shape[-1])
        assert torch.allclose(y, ref, rtol=1e-5, atol=1e-5)
        gy = torch.randn_like(y)
        gx, gw = torch.autograd.grad(y, (x, fc.weight), gy, retain_graph=True)
        rx, rw = torch.autograd.grad(ref, (x, fc.weight), gy)
        assert torch.allclose(gx, rx, rtol=1e-5, atol=1e-5) and torch.allclose(gw, rw, rtol=1e-4, atol=1e-4)


def test_loss_module_builds_without_gpu_and_checks_its_type():
    neuron = {"theta": 10, "tauSr": 1.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1}
    desc = {"neuron": neuron, "simulation": {"Ts": 1.0, "tSample": 100},
            "training": {"error": {"type": "NumSpikes", "tgtSpikeRegion": {"start": 0, "stop": 100},
                                   "tgtSpikeCount": {True: 20, False: 5}}}}
    error = snn.loss(desc)
    assert error.slayer.srmKernel.numel() == 8
    with pytest.raises(AssertionError, match="SpikeTime"):
        error.spikeTime(torch.zeros(1, 1, 1, 1, 100), torch.zeros(1, 1, 1, 1, 100))


def test_dropin_modules_re_export_the_extension_api():
    import importlib
    import sys
    sys.path.insert(0, os.path.join(ROOT, "slayerpytorch_amd", "dropin"))
    try:
        sc = importlib.import_module("slayerCuda")
        slc = importlib.import_module("slayerLoihiCuda")
    finally:
        sys.path.pop(0)
        sys.modules.pop("slayerCuda", None)
        sys.modules.pop("slayerLoihiCuda", None)
    for name in ("getSpikes", "conv", "corr", "shift"):
        assert getattr(sc, name) is getattr(slayerCuda, name)
    assert slc.getSpikes is slayerLoihiCuda.getSpikes


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0 and "one GPU" in (r.stderr + r.stdout)


def test_synapse_and_event_wrappers_need_the_gpu():
    """No CPU path: the synapse ops and the event binning reject CPU tensors before any launch."""
    import slayerpytorch_amd as snn
    from slayerpytorch_amd import synapse
    x, w = torch.zeros((1, 2, 5, 5, 4)), torch.zeros((3, 2, 3, 3))
    with pytest.raises(RuntimeError):
        slayerCuda.getSpikesDelayed(torch.zeros((1, 2, 1, 1, 8)), torch.zeros(3), 10.0, 1.0, 2.0)
    with pytest.raises(RuntimeError):
        slayerCuda.spikeBackwardDelayed(torch.zeros((1, 2, 1, 1, 8)), torch.zeros((1, 2, 1, 1, 8)), 10.0, 10.0, 1.0, 2.0)
    with pytest.raises(RuntimeError):
        synapse.conv(x, w)
    with pytest.raises(RuntimeError):
        synapse.convGradInput(torch.zeros((1, 3, 3, 3, 4)), w, x.shape)
    with pytest.raises(RuntimeError):
        synapse.convGradWeight(torch.zeros((1, 3, 3, 3, 4)), x, w.shape)
    layer = snn.layer({"theta": 10, "tauSr": 1.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1},
                      {"Ts": 1.0, "tSample": 10})
    for mod in (layer.conv(2, 3, 3), layer.pool(2), layer.convTranspose(2, 3, 3), layer.unpool(2)):
        with pytest.raises(RuntimeError):
            mod(torch.zeros((1, 2, 6, 6, 4)))
    assert layer.conv(2, 3, (3, 2), stride=(2, 1), padding=1).weight.shape == (3, 2, 3, 2, 1)
    assert float(layer.pool(2).weight.flatten()[0]) == pytest.approx(11.0)
    with pytest.raises(RuntimeError):
        snn.io.event([1], [1], [0], [1.0]).toSpikeTensor(torch.zeros((1, 4, 4, 8)))


def test_event_class_decodes_like_the_oracle():
    """Host-side members of an event read from file bytes (x, y, p shifted to start at 0, t in ms)."""
    import os
    import slayerpytorch_amd as snn
    from oracle import oracle as O
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "spike_events.npz"))
    for key, fmt in (("nmnist_bs2", 2), ("ntidigits_bs1", 1), ("sample_bs3", 3)):
        ev = snn.io.event._fromBytes(g[key], fmt)
        x, y, p, t = O.decode_events(g[key], fmt)
        assert np.array_equal(ev.x, x) and np.array_equal(ev.p, p - p.min()) and np.array_equal(ev.t, t / 1000)
        assert ev.dim == (1 if fmt == 1 else 2)
        if fmt != 1:
            assert np.array_equal(ev.y, y)


def test_dropout_and_replicate_in_time():
    """Dropout zeroes whole time rows (src/slayer.py:748-759); replicateInTime repeats along T."""
    layer = snn.layer({"theta": 10, "tauSr": 1.0, "tauRef": 1.0, "scaleRef": 2, "tauRho": 1, "scaleRho": 1},
                      {"Ts": 1.0, "tSample": 10})
    torch.manual_seed(0)
    y = layer.dropout(0.5)(torch.ones(4, 3, 5, 5, 10))
    sums = y.sum(-1).flatten()
    assert set(sums.tolist()) == {0.0, 20.0}
    x = torch.rand(2, 3, 4, 4)
    r = layer.replicateInTime(x)
    assert r.shape == (2, 3, 4, 4, 10) and torch.equal(r[..., 7], x)


def test_synapse_geometries_beyond_the_kernels_fall_back_to_torch():
    """The synapse kernels index a filter window of less than 16 MiB and batch items below 2 GiB; the decision is
    made on the host from the sizes alone, and the differentiable ops then call torch's conv3d /
    conv_transpose3d like the reference's layers do (here on CPU tensors: the fallback never reaches the
    library).  Geometries within the limits keep the kernels - and reject CPU tensors."""
    import torch.nn.functional as F
    from slayerpytorch_amd import synapse
    assert synapse.supported((12, 2, 34, 34, 300), (16, 2, 5, 5), 1, 2)
    assert not synapse.supported((1, 2, 346, 260, 5000), (8, 2, 5, 5), 1, 2)          # 5 rows of 346 x 5000 samples
    assert not synapse.supported((1, 16, 128, 128, 8192), (16, 16, 3, 3), 1, 1)       # 4 GiB per batch item
    # a small tensor whose dilated, padded window is 24.6 MB
    geo = dict(stride=1, padding=(1000, 0), dilation=(1000, 1), groups=1)
    x = torch.randn((1, 1, 4, 64, 32), requires_grad=True)
    w = torch.randn((2, 1, 2, 3, 1), requires_grad=True)
    assert not synapse.supported(x.shape, w.shape, **geo)
    y = synapse.synapseConv(x, w, **geo)
    want = F.conv3d(x, w, None, (1, 1, 1), (1000, 0, 0), (1000, 1, 1), 1)
    assert torch.equal(y, want) and y.shape == (1, 2, 1004, 62, 32)
    y.sum().backward()
    assert x.grad is not None and w.grad is not None and float(w.grad.abs().sum()) > 0
    # the transposed op of the same geometry
    z = torch.randn((1, 2, 1004, 62, 32))
    t = synapse.synapseConvTranspose(z, w.detach(), **geo)
    assert torch.equal(t, F.conv_transpose3d(z, w.detach(), None, (1, 1, 1), (1000, 0, 0), 0, 1, (1000, 1, 1)))
    assert t.shape == x.shape
    with pytest.raises(RuntimeError, match="CUDA"):
        synapse.synapseConv(torch.zeros((1, 2, 5, 5, 4)), torch.zeros((3, 2, 3, 3)), 1, 1)

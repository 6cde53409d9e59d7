"""Spike event decoding and binning on the GPU against the CPU oracle: bit-exact (byte and integer
work; the one double-precision rounding is IEEE on both sides)."""
import os

import numpy as np
import pytest
import torch

from oracle import oracle as O
import slayerpytorch_amd as snn
from slayerpytorch_amd import _lib

pytestmark = pytest.mark.gpu

GOLD = np.load(os.path.join(os.path.dirname(__file__), "golden", "spike_events.npz"))


def oracle_tensor(raw, fmt, shape, Ts, shift=0, mode="OR", base=None):
    x, y, p, t = O.decode_events(raw, fmt)
    base = np.zeros(shape, np.float32) if base is None else base
    if x.size == 0:
        return base.copy()
    return O.bin_events(base, x, None if fmt == 1 else y, p - p.min(), t / 1000, Ts, shift, mode)


def random_events(rng, fmt, n, W, H, C, tMaxUs):
    """Packed events with coordinates that partly fall outside a (C, H, W) tensor, repeated bins and
    times exactly half way between two bins."""
    x = rng.integers(0, W + 3, n)
    y = rng.integers(0, H + 3, n)
    t = rng.integers(0, tMaxUs, n)
    t[::7] = (t[::7] // 1000) * 1000 + 500          # .5 ms: rounds to the even bin
    t[::11] = t[0]                                  # shared bins
    out = np.zeros((n, 7 if fmt == 3 else 5), dtype=np.uint8)
    if fmt == 3:
        p = rng.integers(2, C + 4, n)               # channel ids that do not start at 0
        out[:, 0] = x >> 4
        out[:, 1] = ((x << 4) & 0xF0) | ((y >> 8) & 0x0F)
        out[:, 2] = y & 0xFF
        out[:, 3] = p
        out[:, 4], out[:, 5], out[:, 6] = (t >> 16) & 0xFF, (t >> 8) & 0xFF, t & 0xFF
    else:
        p = rng.integers(0, 2, n)
        if fmt == 1:
            out[:, 0], out[:, 1] = x >> 8, x & 0xFF
        else:
            out[:, 0], out[:, 1] = x, y
        out[:, 2] = ((t >> 16) & 0x7F) | (p << 7)
        out[:, 3], out[:, 4] = (t >> 8) & 0xFF, t & 0xFF
    return out.reshape(-1)


@pytest.mark.parametrize("Ts,T", [(1.0, 350), (2.0, 175), (0.5, 300), (3.0, 40)])
def test_nmnist_sample_from_file_bytes(Ts, T):
    raw = GOLD["nmnist_bs2"]
    ev = snn.io.event._fromBytes(raw, 2)
    got = ev.toSpikeTensor(torch.zeros((2, 34, 34, T), device="cuda"), samplingTime=Ts).cpu().numpy()
    ref = oracle_tensor(raw, 2, (2, 34, 34, T), Ts)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    assert got.sum() > 0


def test_nmnist_sample_matches_reference_rasters():
    """The reference's own binned rasters of this sample (1 ms and 2 ms bins, binned by truncation):
    events moved to the start of their bin must reproduce them through the decoded-array path."""
    gold = np.load(os.path.join(os.path.dirname(__file__), "golden", "nmnist_response.npz"))
    x, y, p, t = O.decode_events(GOLD["nmnist_bs2"], 2)
    for Ts, key in ((1, "binned"), (2, "binned_ts2")):
        shape = tuple(gold[key + "_shape"])
        raster = np.zeros(shape, np.float32)
        raster[gold[key + "_events"][:, 0], gold[key + "_events"][:, 1]] = gold[key + "_values"]
        ev = snn.io.event(x, y, p, np.floor(t / 1000 / Ts) * Ts)
        got = ev.toSpikeTensor(torch.zeros((2, 34, 34, shape[1]), device="cuda"), samplingTime=Ts)
        assert np.array_equal(got.cpu().numpy().reshape(shape), raster)


@pytest.mark.parametrize("fmt", [1, 2, 3])
@pytest.mark.parametrize("mode", ["OR", "SUM"])
def test_batch_of_random_samples(fmt, mode):
    rng = np.random.default_rng(100 + fmt)
    C, H, W, T, Ts = (3 if fmt == 3 else 2), (1 if fmt == 1 else 9), 12, 50, 1.5
    counts = [1, 700, 5000, 257]
    raws = [random_events(rng, fmt, n, W, H, C, int(T * Ts * 1000 * 1.2)) for n in counts]
    events = [snn.io.event._fromBytes(r, fmt) for r in raws]
    keep = list(range(len(events)))
    base = rng.standard_normal((len(keep), C, H, W, T)).astype(np.float32)
    got = snn.io.toSpikeTensorBatch([events[i] for i in keep], torch.from_numpy(base).cuda(), Ts, False, mode)
    for k, i in enumerate(keep):
        ref = oracle_tensor(raws[i], fmt, (C, H, W, T), Ts, 0, mode, base[k])
        assert np.array_equal(got[k].cpu().numpy().view(np.uint32), ref.view(np.uint32)), "sample %d" % i


def test_time_shift_and_large_sample():
    """A sample large enough for several work-groups, with the reference's random start bin."""
    rng = np.random.default_rng(5)
    raw = random_events(rng, 2, 60000, 34, 34, 2, 400000)
    ev = snn.io.event._fromBytes(raw, 2)
    np.random.seed(3)
    got = ev.toSpikeTensor(torch.zeros((2, 34, 34, 100), device="cuda"), 1.0, randomShift=True)
    np.random.seed(3)
    shift = ev._shift(1.0, 100, True)
    assert shift > 0
    ref = oracle_tensor(raw, 2, (2, 34, 34, 100), 1.0, shift)
    assert np.array_equal(got.cpu().numpy(), ref)


def test_decoded_arrays_path():
    rng = np.random.default_rng(8)
    n = 3000
    x, y, p = rng.integers(-2, 20, n), rng.integers(-2, 12, n), rng.integers(1, 4, n)
    t = rng.random(n) * 70 - 2
    t[::5] = np.floor(t[::5]) + 0.5
    ev = snn.io.event(x, y, p, t)
    base = rng.standard_normal((3, 10, 16, 64)).astype(np.float32)
    for mode in ("OR", "SUM"):
        got = ev.toSpikeTensor(torch.from_numpy(base).cuda(), 0.75, False, mode).cpu().numpy()
        ref = O.bin_events(base, ev.x, ev.y, ev.p, ev.t, 0.75, 0, mode)
        assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))
    one = snn.io.event(x, None, p, t)                                   # one spatial dimension
    got = one.toSpikeTensor(torch.zeros((3, 1, 16, 64), device="cuda"), 1.0).cpu().numpy()
    assert np.array_equal(got, O.bin_events(np.zeros((3, 1, 16, 64), np.float32), one.x, None, one.p, one.t, 1.0))


def test_events_changed_after_reading_are_binned_as_changed():
    # an augmentation between read and bin (a flip, a time offset): the members are binned, as in the reference,
    # not the file's bytes
    raw, shape = GOLD["nmnist_bs2"], (2, 34, 34, 350)
    x, y, p, t = O.decode_events(raw, 2)
    want = O.bin_events(np.zeros(shape, np.float32), 33 - x, y, p - p.min(), t / 1000 + 20.0, 1.0)
    same = snn.io.event._fromBytes(raw, 2).toSpikeTensor(torch.zeros(shape, device="cuda"), 1.0).cpu().numpy()
    assert not np.array_equal(want, same)
    ev = snn.io.event._fromBytes(raw, 2)             # new arrays assigned
    ev.x = 33 - ev.x
    ev.t = ev.t + 20.0
    assert np.array_equal(ev.toSpikeTensor(torch.zeros(shape, device="cuda"), 1.0).cpu().numpy(), want)
    ev = snn.io.event._fromBytes(raw, 2)             # the same edits in place, as the reference's writable arrays allow
    assert ev._packed() == 2
    ev.x[:] = 33 - ev.x
    ev.t += 20.0
    assert np.array_equal(ev.toSpikeTensor(torch.zeros(shape, device="cuda"), 1.0).cpu().numpy(), want)
    assert ev._packed() is None
    ev = snn.io.event._fromBytes(raw, 2)             # a single element
    ev.p[7] = 1 - ev.p[7]
    pp = p - p.min()
    pp[7] = 1 - pp[7]
    assert np.array_equal(ev.toSpikeTensor(torch.zeros(shape, device="cuda"), 1.0).cpu().numpy(),
                          O.bin_events(np.zeros(shape, np.float32), x, y, pp, t / 1000, 1.0))


def test_argument_errors():
    lib = _lib.load()
    t = torch.zeros((2, 4, 4, 8), device="cuda")
    assert lib.slayer_bin_events_f32(t.data_ptr(), None, None, None, None, None, 5, 0, 2, 4, 4, 8, 1.0, 0, None) == 1
    assert lib.slayer_bin_events_f32(t.data_ptr(), None, None, None, None, None, 0, 0, 2, 4, 4, 8, 1.0, 0, None) == 0
    assert lib.slayer_bin_events_f32(t.data_ptr(), None, None, None, None, None, 5, 0, 2, 4, 4, 8, 0.0, 0, None) == 1
    assert lib.slayer_bin_packed_events_f32(t.data_ptr(), None, None, 10, None, 1, 2, 7, 2, 4, 4, 8, 1.0, 0, None) == 1
    # a table entry that points outside the byte buffer is skipped, not read
    raw = torch.zeros(10, dtype=torch.uint8, device="cuda")
    table = torch.tensor([[5, 100, 0]], dtype=torch.int64, device="cuda")
    assert lib.slayer_bin_packed_events_f32(t.data_ptr(), None, raw.data_ptr(), 10, table.data_ptr(), 1, 100, 2, 2, 4, 4,
                                            8, 1.0, 0, None) == 0
    torch.cuda.synchronize()
    assert float(t.abs().sum()) == 0.0
    with pytest.raises(RuntimeError):
        snn.io.event([1], [1], [0], [1.0]).toSpikeTensor(torch.zeros((2, 4, 4, 8)))


def test_binning_on_a_side_stream():
    """Upload and binning run on PyTorch's current stream: under a side stream they can overlap other
    work, and the result is the same once that stream is waited for."""
    raw = GOLD["nmnist_bs2"]
    events = [snn.io.event._fromBytes(raw, 2) for _ in range(3)]
    side = torch.cuda.Stream()
    busy = torch.randn((2048, 2048), device="cuda")
    with torch.cuda.stream(side):
        out = snn.io.toSpikeTensorBatch(events, torch.zeros((3, 2, 34, 34, 350), device="cuda"), 1.0)
    for _ in range(4):
        busy = busy @ busy * 1e-3                     # work on the default stream meanwhile
    torch.cuda.current_stream().wait_stream(side)
    ref = oracle_tensor(raw, 2, (2, 34, 34, 350), 1.0)
    for k in range(3):
        assert np.array_equal(out[k].cpu().numpy(), ref)

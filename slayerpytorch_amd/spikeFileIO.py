"""Spike event files and their conversion to spike tensors (src/spikeFileIO.py), with the
conversion done on the GPU.

The reference decodes a sample's event file with numpy and bins it into a dense (C, H, W, T)
tensor in a data-loader worker (``read2Dspikes(file).toSpikeTensor(torch.zeros(...))``,
src/spikeFileIO.py:233-259 and :66-144); the dense tensor then crosses PCIe.  Here the file's
bytes go to the device as they are and one kernel decodes and bins them, for one sample
(``event.toSpikeTensor``) or for a whole batch in a single launch (``toSpikeTensorBatch``).  The
tensor to fill must live on the GPU; there is no host implementation of the binning.

``event`` keeps the reference's members ``x``, ``y``, ``p``, ``t`` (numpy arrays, decoded on first
use when the event came from a file) and ``dim``.
"""
import numpy as np
import torch

from . import _lib
from .slayerCuda import _on_device_of, _ptr

__all__ = ["event", "read1Dspikes", "read2Dspikes", "read3Dspikes", "toSpikeTensorBatch"]

_EVENT_BYTES = {1: 5, 2: 5, 3: 7}
_MODES = {"OR": 0, "SUM": 1}


def _decode(raw, fmt):
    """numpy view of the packed events: x, y (None for 1-D files), p, t in microseconds."""
    b = raw.reshape(-1, _EVENT_BYTES[fmt]).astype(np.int64)
    if fmt == 3:
        x = (b[:, 0] << 4) | (b[:, 1] >> 4)
        y = b[:, 2] | ((b[:, 1] & 0x0F) << 8)
        p = b[:, 3]
        t = (b[:, 4] << 16) | (b[:, 5] << 8) | b[:, 6]
        return x, y, p, t
    t = ((b[:, 2] << 16) | (b[:, 3] << 8) | b[:, 4]) & 0x7FFFFF
    p = b[:, 2] >> 7
    if fmt == 1:
        return (b[:, 0] << 8) | b[:, 1], None, p, t
    return b[:, 0], b[:, 1], p, t


class event():
    """Spike events ``x``, ``y`` (``None`` for one spatial dimension), polarity / channel ``p``
    and time stamps ``t`` in ms (src/spikeFileIO.py:6-34).  As in the reference the polarity is
    shifted so that its minimum is 0."""

    # The events of a file are binned from the file's bytes (one launch decodes and bins a whole batch) for as long as
    # nobody outside this module has touched the decoded arrays: x, y, p and t are properties over private members,
    # and reading one of them - the only way to edit it in place, ev.t -= ev.t.min(), ev.x[:] = W - 1 - ev.x - or
    # assigning a new array makes the members what is binned from then on, as in the reference.  The arrays
    # themselves are ordinary writable arrays.
    def _touched(self):
        self._raw = None
        self._format = None

    def _member(name):
        def get(self):
            self._touched()
            return getattr(self, "_" + name)

        def put(self, value):
            self._touched()
            setattr(self, "_" + name, value)
        return property(get, put)

    x, y, p, t = _member("x"), _member("y"), _member("p"), _member("t")
    del _member

    def __init__(self, xEvent, yEvent, pEvent, tEvent):
        self._raw = None
        self._format = None
        self.dim = 1 if yEvent is None else 2
        self._x = np.asarray(xEvent)
        self._y = yEvent if yEvent is None else np.asarray(yEvent)
        self._p = np.asarray(pEvent)
        self._t = np.asarray(tEvent)
        if not issubclass(self._x.dtype.type, np.integer):
            self._x = self._x.astype("int")
        if not issubclass(self._p.dtype.type, np.integer):
            self._p = self._p.astype("int")
        if self.dim == 2 and not issubclass(self._y.dtype.type, np.integer):
            self._y = self._y.astype("int")
        self._p = self._p - self._p.min()

    @classmethod
    def _fromBytes(cls, raw, fmt):
        raw = np.ascontiguousarray(raw, dtype=np.uint8)
        n = raw.size // _EVENT_BYTES[fmt]
        raw = raw[:n * _EVENT_BYTES[fmt]]
        x, y, p, t = _decode(raw, fmt)
        self = cls(x, y, p, t / 1000)          # spike times in ms
        self._raw, self._format = raw, fmt
        return self

    def _packed(self):
        """The layout of the file bytes while they still describe the events, else None."""
        return self._format

    def _shift(self, samplingTime, T, randomShift):
        """The reference's random start bin (src/spikeFileIO.py:80-90), drawn on the host."""
        if randomShift is not True:
            return 0
        return int(np.random.randint(max(int(self._t.min() / samplingTime),
                                         int(self._t.max() / samplingTime) - T,
                                         T - int(self._t.max() / samplingTime), 1)))

    def toSpikeTensor(self, emptyTensor, samplingTime=1, randomShift=False, binningMode="OR"):
        """Bins the events into ``emptyTensor`` (C, H, W, T), a float32 tensor on the GPU, in place,
        and returns it (src/spikeFileIO.py:66-144): bin = round(t / samplingTime), events outside the
        tensor are dropped, 'OR' stores ``1/samplingTime``, 'SUM' adds it once per occupied bin."""
        _check_tensor(emptyTensor, 4)
        return toSpikeTensorBatch([self], emptyTensor.unsqueeze(0), samplingTime, randomShift, binningMode)[0]


def _check_tensor(t, dims):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise RuntimeError("the tensor to fill must be a CUDA tensor (the events are binned on the GPU)")
    if t.dtype != torch.float32 or not t.is_contiguous() or t.dim() != dims:
        raise RuntimeError("expected a contiguous float32 tensor with %d dimensions" % dims)


def toSpikeTensorBatch(events, emptyTensor, samplingTime=1, randomShift=False, binningMode="OR"):
    """Bins ``events[i]`` into ``emptyTensor[i]`` for a batch: ``emptyTensor`` is (N, C, H, W, T) on
    the GPU.  Events read from files of one layout are decoded and binned by a single launch from
    their file bytes; other events are uploaded as decoded arrays, one launch per sample."""
    _check_tensor(emptyTensor, 5)
    if len(events) != emptyTensor.shape[0]:
        raise RuntimeError("%d event sets for a batch of %d" % (len(events), emptyTensor.shape[0]))
    if binningMode.upper() not in _MODES:
        raise Exception("Unsupported binningMode. It was {}".format(binningMode))
    mode = _MODES[binningMode.upper()]
    N, C, H, W, T = emptyTensor.shape
    lib = _lib.load()
    base = emptyTensor.clone() if mode == 1 else None
    shifts = [ev._shift(samplingTime, T, randomShift) for ev in events]
    formats = {ev._packed() for ev in events}
    packed = None not in formats and len(formats) == 1 and all(ev.dim == (1 if ev._format == 1 else 2) for ev in events)
    if packed and events[0]._format == 1 and H != 1:
        raise RuntimeError("1-D events need a tensor of height 1, got %d" % H)
    with _on_device_of(emptyTensor) as stream:
        if packed and N > 0:
            fmt = events[0]._format
            table, first = np.zeros((N, 3), dtype=np.int64), 0
            for i, ev in enumerate(events):
                table[i] = (first, ev._raw.size // _EVENT_BYTES[fmt], shifts[i])
                first += ev._raw.size
            # one upload: the sample table followed by the files' bytes, staged in pinned host memory
            # (allocated pinned by PyTorch's caching host allocator) so that the copy is asynchronous
            staging = torch.empty(table.nbytes + first, dtype=torch.uint8, pin_memory=True)
            host = staging.numpy()
            host[:table.nbytes] = table.reshape(-1).view(np.uint8)
            at = table.nbytes
            for ev in events:
                host[at:at + ev._raw.size] = ev._raw
                at += ev._raw.size
            d_staging = staging.to(emptyTensor.device, non_blocking=True)
            _lib.check(lib.slayer_bin_packed_events_f32(
                _ptr(emptyTensor), _ptr(base) if base is not None else None, d_staging.data_ptr() + table.nbytes, first,
                d_staging.data_ptr(), N, int(table[:, 1].max()), fmt, C, H, W, T, float(samplingTime), mode, stream),
                "slayer_bin_packed_events_f32")
            return emptyTensor
        for i, ev in enumerate(events):
            if ev.dim == 1 and H != 1:
                raise RuntimeError("1-D events need a tensor of height 1, got %d" % H)
            dev = emptyTensor.device
            x = torch.from_numpy(np.ascontiguousarray(ev._x, dtype=np.int32)).to(dev)
            p = torch.from_numpy(np.ascontiguousarray(ev._p, dtype=np.int32)).to(dev)
            t = torch.from_numpy(np.ascontiguousarray(ev._t, dtype=np.float64)).to(dev)
            y = None if ev.dim == 1 else torch.from_numpy(np.ascontiguousarray(ev._y, dtype=np.int32)).to(dev)
            _lib.check(lib.slayer_bin_events_f32(
                _ptr(emptyTensor[i]), _ptr(base[i]) if base is not None else None, _ptr(x),
                _ptr(y) if y is not None else None, _ptr(p), _ptr(t), x.numel(), shifts[i], C, H, W, T,
                float(samplingTime), mode, stream), "slayer_bin_events_f32")
    return emptyTensor


def _read(filename, fmt):
    return event._fromBytes(np.fromfile(filename, dtype=np.uint8), fmt)


def read1Dspikes(filename):
    """Events of a one-dimensional binary spike file: 40 bits per event, 16-bit neuron id,
    polarity bit, 23-bit time stamp in microseconds (src/spikeFileIO.py:162-184)."""
    return _read(filename, 1)


def read2Dspikes(filename):
    """Events of a two-dimensional binary spike file (the NMNIST / NCALTECH101 layout): 40 bits
    per event, 8-bit x, 8-bit y, polarity bit, 23-bit time stamp in microseconds
    (src/spikeFileIO.py:233-259)."""
    return _read(filename, 2)


def read3Dspikes(filename):
    """Events of a binary spike file with a channel dimension: 56 bits per event, 12-bit x,
    12-bit y, 8-bit channel, 24-bit time stamp in microseconds (src/spikeFileIO.py:296-321)."""
    return _read(filename, 3)

"""numpy front-end of the CPU oracle (``slayer_oracle.c``).

TEST INFRASTRUCTURE ONLY: the tests, the smoke check and the benchmark's ``cpu_baseline``
leg import this module as the checker.  The product package never does, and it has no CPU
fallback: without the HIP library it raises.

Each function takes and returns C-contiguous ``float32`` numpy arrays whose last axis is
time, exactly like the extension entry points they mirror:

=====================  ==========================================================
oracle function        reference entry point it restates
=====================  ==========================================================
``get_spikes``         ``slayerCuda.getSpikes``  (src/cuda/slayerKernels.cu:14-39)
``conv`` / ``corr``    ``slayerCuda.conv/corr``  (src/cuda/slayerKernels.cu:41-75)
``shift``              ``slayerCuda.shift``      (src/cuda/slayerKernels.cu:77-134)
``loihi_get_spikes``   ``slayerLoihiCuda.getSpikes`` (src/cuda/slayerLoihiKernels.cu:12-46)
``spike_bwd``          ``_spikeFunction.backward`` (src/slayer.py:857-865)
``delay_grad``         ``_delayFunction.backward`` (src/slayer.py:949-955)
``decode_events``      ``spikeFileIO.read1Dspikes/read2Dspikes/read3Dspikes`` (src/spikeFileIO.py:162-321)
``bin_events``         ``spikeFileIO.event.toSpikeTensor`` (src/spikeFileIO.py:66-144)
``synapse_conv*``      ``F.conv3d`` with a (KH, KW, 1) kernel in the synapse layers
                       (src/slayer.py:499-507, :565-575) and its two gradients
=====================  ==========================================================
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libslayer_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_i64 = ctypes.c_int64


class SynapseGeom(ctypes.Structure):
    """Geometry of a per-timestep 2-D synapse: input [N][C][H][W][T], weights [O][C/groups][KH][KW]."""
    _fields_ = [(k, ctypes.c_int32) for k in ("N", "C", "H", "W", "T", "O", "KH", "KW", "sH", "sW",
                                              "pH", "pW", "dH", "dW", "groups")]


def build(force=False):
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force:
        subprocess.run(["make", "-C", _HERE, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", _HERE], check=True, stdout=subprocess.DEVNULL)


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.oracle_set_threads.argtypes = [ctypes.c_int]
        L.oracle_get_threads.restype = ctypes.c_int
        L.oracle_max_threads.restype = ctypes.c_int
        L.oracle_get_spikes_f32.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64,
                                            ctypes.c_float, ctypes.c_float]
        for fn in (L.oracle_conv_f32, L.oracle_corr_f32):
            fn.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64, ctypes.c_float, ctypes.c_int]
        L.oracle_shift_f32.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64, _i64, ctypes.c_float]
        L.oracle_spike_bwd_f32.argtypes = [_f32p, _f32p, _f32p, ctypes.c_float, ctypes.c_float,
                                           ctypes.c_float, _i64]
        L.oracle_delay_grad_f32.argtypes = [_f32p, _f32p, _f32p, _i64, _i64, _i64, ctypes.c_float]
        L.oracle_loihi_get_spikes_f32.argtypes = [_f32p, _f32p, _f32p, _f32p, _i64, _i64,
                                                  ctypes.c_uint32, ctypes.c_int32, ctypes.c_uint32,
                                                  ctypes.c_uint32, ctypes.c_uint32]
        gp = ctypes.POINTER(SynapseGeom)
        L.oracle_synapse_out_shape.argtypes = [gp, ctypes.POINTER(_i64), ctypes.POINTER(_i64)]
        L.oracle_synapse_conv_f32.argtypes = [_f32p, _f32p, _f32p, gp]
        L.oracle_synapse_conv_grad_input_f32.argtypes = [_f32p, _f32p, _f32p, gp]
        L.oracle_synapse_conv_grad_weight_f32.argtypes = [_f32p, _f32p, _f32p, gp]
        for name in ("oracle_synapse_out_shape", "oracle_synapse_conv_f32",
                     "oracle_synapse_conv_grad_input_f32", "oracle_synapse_conv_grad_weight_f32"):
            getattr(L, name).restype = None
        i32p, u8p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_uint8)
        f64p = ctypes.POINTER(ctypes.c_double)
        L.oracle_decode_events.argtypes = [i32p, i32p, i32p, i32p, u8p, _i64, ctypes.c_int32]
        L.oracle_decode_events.restype = None
        L.oracle_bin_events_f32.argtypes = [_f32p, _f32p, i32p, i32p, i32p, f64p, _i64, _i64] + \
            [ctypes.c_int32] * 4 + [ctypes.c_double, ctypes.c_int32]
        L.oracle_bin_events_f32.restype = None
        for name in ("oracle_get_spikes_f32", "oracle_conv_f32", "oracle_corr_f32",
                     "oracle_shift_f32", "oracle_spike_bwd_f32", "oracle_delay_grad_f32",
                     "oracle_loihi_get_spikes_f32", "oracle_set_threads"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def set_threads(n):
    """Host threads for the per-neuron loop (results do not depend on it)."""
    lib().oracle_set_threads(int(n))


def max_threads():
    return lib().oracle_max_threads()


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a


def _p(a):
    return a.ctypes.data_as(_f32p)


def _rows(a):
    T = a.shape[-1]
    return (a.size // T if T else 0), T


def get_spikes(u, nu, theta, Ts):
    """Returns ``(spikes, u_after)``; ``u`` itself is left untouched (a copy is mutated)."""
    u = _f32(u).copy()
    nu = _f32(nu).reshape(-1)
    s = np.empty_like(u)
    n, T = _rows(u)
    if u.size:
        lib().oracle_get_spikes_f32(_p(s), _p(u), _p(nu), n, T, nu.size, float(theta), float(Ts))
    return s, u


def _fir(fn, x, filt, Ts, fused):
    x = _f32(x)
    filt = _f32(filt).reshape(-1)
    out = np.empty_like(x)
    n, T = _rows(x)
    if x.size:
        fn(_p(out), _p(x), _p(filt), n, T, filt.size, float(Ts), int(bool(fused)))
    return out


def conv(x, filt, Ts, fused=True):
    """Causal FIR along the last axis; ``fused`` selects fmaf accumulation."""
    return _fir(lib().oracle_conv_f32, x, filt, Ts, fused)


def corr(x, filt, Ts, fused=True):
    """Anti-causal FIR (adjoint of :func:`conv`) along the last axis."""
    return _fir(lib().oracle_corr_f32, x, filt, Ts, fused)


def shift(x, delay, Ts=1.0):
    """``delay``: a number / one-element array (all rows) or an array with one entry per
    neuron of a batch item (``x.size / T / x.shape[0]`` entries, shared by every batch item)."""
    x = _f32(x)
    lut = _f32(np.asarray(delay, dtype=np.float32)).reshape(-1)
    out = np.empty_like(x)
    n, T = _rows(x)
    if lut.size == 1:
        nb, per = 1, n
    else:
        nb = x.shape[0]
        per = n // nb
        if lut.size != per:
            raise ValueError("shift and number of neurons must be same")
    if x.size:
        lib().oracle_shift_f32(_p(out), _p(x), _p(lut), lut.size, nb, per, T, float(Ts))
    return out


def spike_bwd(grad_out, u, theta, tau, scale):
    """``tau`` is the already scaled time constant ``tauRho * theta``."""
    g = _f32(grad_out)
    u = _f32(u)
    out = np.empty_like(g)
    if g.size:
        lib().oracle_spike_bwd_f32(_p(out), _p(g), _p(u), float(theta), float(tau), float(scale),
                                   g.size)
    return out


def delay_grad(out, grad_out, Ts):
    """Gradient w.r.t. a per-neuron delay table; result has shape ``out.shape[1:-1]``."""
    y = _f32(out)
    g = _f32(grad_out)
    nb = y.shape[0]
    n, T = _rows(y)
    per = n // nb
    res = np.zeros(per, dtype=np.float32)
    if y.size:
        lib().oracle_delay_grad_f32(_p(res), _p(y), _p(g), nb, per, T, float(Ts))
    return res.reshape(y.shape[1:-1])


def loihi_get_spikes(w, wgtExp, theta, iDecay, vDecay, refDelay):
    """Returns ``(spike, voltage, current)`` like ``slayerLoihiCuda.getSpikes``."""
    if int(refDelay) < 1:
        raise ValueError("refDelay must be >= 1")
    w = _f32(w)
    s = np.empty_like(w)
    v = np.empty_like(w)
    u = np.empty_like(w)
    n, T = _rows(w)
    if w.size:
        lib().oracle_loihi_get_spikes_f32(_p(s), _p(v), _p(u), _p(w), n, T, int(wgtExp), int(theta),
                                          int(iDecay), int(vDecay), int(refDelay))
    return s, v, u


def _pair(v):
    return (int(v), int(v)) if np.isscalar(v) else (int(v[0]), int(v[1]))


def synapse_geom(in_shape, w_shape, stride=1, padding=0, dilation=1, groups=1):
    """Geometry record and output shape of the synapse ``in_shape`` = (N, C, H, W, T),
    ``w_shape`` = (O, C/groups, KH, KW[, 1])."""
    N, C, H, W, T = (int(v) for v in in_shape)
    O, Cg, KH, KW = (int(v) for v in w_shape[:4])
    if C % groups or O % groups or Cg != C // groups:
        raise ValueError("channels and groups do not fit the weight shape")
    (sH, sW), (pH, pW), (dH, dW) = _pair(stride), _pair(padding), _pair(dilation)
    g = SynapseGeom(N, C, H, W, T, O, KH, KW, sH, sW, pH, pW, dH, dW, int(groups))
    OH, OW = _i64(), _i64()
    lib().oracle_synapse_out_shape(ctypes.byref(g), ctypes.byref(OH), ctypes.byref(OW))
    return g, (N, O, OH.value, OW.value, T)


def synapse_conv(x, w, stride=1, padding=0, dilation=1, groups=1):
    """Per-timestep 2-D cross-correlation of ``x`` [N][C][H][W][T] with ``w`` [O][C/groups][KH][KW]."""
    x, w = _f32(x), _f32(w)
    g, oshape = synapse_geom(x.shape, w.shape, stride, padding, dilation, groups)
    out = np.zeros(oshape, dtype=np.float32)
    if out.size:
        lib().oracle_synapse_conv_f32(_p(out), _p(x), _p(w), ctypes.byref(g))
    return out


def synapse_conv_grad_input(grad_out, w, in_shape, stride=1, padding=0, dilation=1, groups=1):
    """Gradient of :func:`synapse_conv` with respect to ``x`` (shape ``in_shape``)."""
    go, w = _f32(grad_out), _f32(w)
    g, oshape = synapse_geom(in_shape, w.shape, stride, padding, dilation, groups)
    if tuple(go.shape) != oshape:
        raise ValueError("grad_out has shape %s, expected %s" % (go.shape, oshape))
    gi = np.zeros(tuple(int(v) for v in in_shape), dtype=np.float32)
    if gi.size:
        lib().oracle_synapse_conv_grad_input_f32(_p(gi), _p(go), _p(w), ctypes.byref(g))
    return gi


def synapse_conv_grad_weight(grad_out, x, w_shape, stride=1, padding=0, dilation=1, groups=1):
    """Gradient of :func:`synapse_conv` with respect to ``w`` (shape ``w_shape[:4]``)."""
    go, x = _f32(grad_out), _f32(x)
    g, oshape = synapse_geom(x.shape, w_shape, stride, padding, dilation, groups)
    if tuple(go.shape) != oshape:
        raise ValueError("grad_out has shape %s, expected %s" % (go.shape, oshape))
    gw = np.zeros(tuple(int(v) for v in w_shape[:4]), dtype=np.float32)
    if gw.size:
        lib().oracle_synapse_conv_grad_weight_f32(_p(gw), _p(go), _p(x), ctypes.byref(g))
    return gw


def decode_events(data, fmt):
    """``(x, y, p, tUs)`` int32 arrays of the packed events in ``data`` (bytes / uint8 array);
    ``fmt`` 1, 2 or 3 for the 1-D, 2-D and 3-D file layouts.  The polarity is the stored one
    (not yet shifted to start at 0)."""
    b = np.ascontiguousarray(np.frombuffer(bytes(data), dtype=np.uint8))
    n = b.size // (7 if fmt == 3 else 5)
    out = [np.zeros(n, dtype=np.int32) for _ in range(4)]
    i32p, u8p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_uint8)
    if n:
        lib().oracle_decode_events(*[a.ctypes.data_as(i32p) for a in out], b.ctypes.data_as(u8p), n, int(fmt))
    return tuple(out)


def bin_events(tensor, x, y, p, t_ms, sampling_time=1.0, time_shift=0, mode="OR"):
    """Returns a copy of the (C, H, W, T) float32 ``tensor`` with the events binned into it."""
    base = _f32(tensor)
    out = base.copy()
    C, H, W, T = out.shape
    x = np.ascontiguousarray(x, dtype=np.int32)
    p = np.ascontiguousarray(p, dtype=np.int32)
    t = np.ascontiguousarray(t_ms, dtype=np.float64)
    i32p, f64p = ctypes.POINTER(ctypes.c_int32), ctypes.POINTER(ctypes.c_double)
    yp = None
    if y is not None:
        y = np.ascontiguousarray(y, dtype=np.int32)
        yp = y.ctypes.data_as(i32p)
    if x.size:
        lib().oracle_bin_events_f32(_p(out), _p(base), x.ctypes.data_as(i32p), yp, p.ctypes.data_as(i32p),
                                    t.ctypes.data_as(f64p), x.size, int(time_shift), C, H, W, T,
                                    float(sampling_time), {"OR": 0, "SUM": 1}[mode.upper()])
    return out

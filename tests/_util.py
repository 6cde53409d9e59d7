"""Shared helpers of the test-suite: golden fixtures and small raster builders."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden(name):
    return np.load(os.path.join(GOLDEN, name))


def raster_from_aer(aer, n_neurons, n_steps, Ts, amplitude, time_first=True, one_based=True, offset=0):
    """Dense (n_neurons, n_steps) raster from an address-event list.

    ``time_first``: rows are (time in ms, neuron id) as in snnData/*.txt; otherwise
    (neuron id, time bin) as in the Loihi recordings.  Events at or after ``n_steps`` are dropped.
    """
    aer = np.asarray(aer, dtype=np.float64)
    out = np.zeros((n_neurons, n_steps), dtype=np.float32)
    for row in aer:
        if time_first:
            t, n = row[0] / Ts + offset, row[1] - (1 if one_based else 0)
        else:
            n, t = row[0], row[1] + offset
        t, n = int(np.rint(t)), int(np.rint(n))
        if t < n_steps:
            out[n, t] = amplitude
    return out


def raster_from_events(shape, events, values):
    out = np.zeros(tuple(int(x) for x in shape), dtype=np.float32)
    out[events[:, 0], events[:, 1]] = values
    return out


def rel_err(a, b):
    """max |a-b| / max |b| (norm-wise relative error)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    scale = np.abs(b).max() if b.size else 1.0
    return float(np.abs(a - b).max() / (scale if scale > 0 else 1.0)) if b.size else 0.0

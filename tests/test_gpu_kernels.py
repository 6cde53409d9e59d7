"""Parity of the HIP kernels with the CPU oracle on the same seeded inputs.  Every call goes
through the Python modules ``slayerCuda`` / ``slayerLoihiCuda``, i.e. ctypes -> C ABI of
libslayer_hip.so.  Integer/threshold work (spike, Loihi, shift) must be bit-exact; fp32 filters
must stay within 1e-5 relative (the chain kernels are in fact bit-exact against the
fused-multiply-add oracle, which is asserted too; the matrix-core correlation is not and is held
to the tolerance).
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from slayerpytorch_amd import _lib, slayerCuda, slayerLoihiCuda
from slayerpytorch_amd.slayer import alphaKernel

from _util import rel_err

pytestmark = pytest.mark.gpu

REL_TOL = 1e-5       # psp / corr / spike pdf / delay gradient: max |gpu - oracle| <= REL_TOL * max |oracle|


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def bits(a):
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


@pytest.fixture(params=[0, 1], ids=["tiled", "generic"])
def impl(request):
    lib = _lib.load()
    old = lib.slayer_force_generic_kernels(request.param)
    yield request.param
    lib.slayer_force_generic_kernels(old)


# ------------------------------------------------------------------------------------------ shift
@pytest.mark.parametrize("shape", [(5, 10, 20, 30, 100), (3, 7, 1, 1, 33), (2, 3, 2, 2, 1), (1, 1, 1, 1, 5000),
                                   (4, 130, 1, 1, 350)])
def test_shift_per_neuron_exact(shape):
    rng = np.random.default_rng(9)
    Ts = 0.1
    x = rng.standard_normal(shape).astype(np.float32)
    d = (rng.random(shape[1:4]) * 2 - 1).astype(np.float32) * shape[-1] * Ts / 4
    d.reshape(-1)[0] = 0.0
    got = host(slayerCuda.shift(dev(x), dev(d), Ts))
    assert np.array_equal(bits(got), bits(O.shift(x, d, Ts)))
    # negated table (backward direction)
    got = host(slayerCuda.shift(dev(x), dev(d), Ts, sign=-1.0))
    assert np.array_equal(bits(got), bits(O.shift(x, -d, Ts)))


@pytest.mark.parametrize("delay,Ts", [(4, 1.0), (-3, 1.0), (0, 1.0), (-0.25, 0.1), (0.3, 0.1), (1000.0, 1.0),
                                      (-1e12, 1.0), (2.5, 0.5)])
@pytest.mark.parametrize("T", [300, 350, 33])
def test_shift_scalar_exact(delay, Ts, T):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 5, 2, 2, T)).astype(np.float32)
    want = O.shift(x, delay, Ts)
    assert np.array_equal(bits(host(slayerCuda.shift(dev(x), delay, Ts))), bits(want))
    # one-element tensor: read on the device, same result
    assert np.array_equal(bits(host(slayerCuda.shift(dev(x), dev(np.array([delay], np.float32)), Ts))), bits(want))
    if Ts == 1.0:
        assert np.array_equal(bits(host(slayerCuda.shift(dev(x), delay))), bits(want))      # Ts defaults to 1


@pytest.mark.parametrize("shape", [(4, 3, 1, 1, 5), (2, 6, 1, 1, 6), (8, 5, 1, 1, 7), (4, 9, 2, 1, 101), (2, 2, 3, 5, 350),
                                   (4, 1, 1, 1, 2001), (1, 4, 1, 1, 4097)])
def test_shift_rows_that_are_not_whole_vectors(shape):
    # T % 4 != 0 with rows * T % 4 == 0: aligned output vectors span two rows with different delays
    rng = np.random.default_rng(shape[-1])
    T = shape[-1]
    x = rng.standard_normal(shape).astype(np.float32)
    d = np.round((rng.random(shape[1:4]) * 2 - 1) * (T + 3)).astype(np.float32)     # up to beyond the row length
    d.reshape(-1)[0] = 0.0
    for sign in (1.0, -1.0):
        got = host(slayerCuda.shift(dev(x), dev(d), 1.0, sign=sign))
        assert np.array_equal(bits(got), bits(O.shift(x, sign * d, 1.0)))
    for delay in (1.0, -1.0, 3.0, float(T - 1), float(T), -float(T + 5), 0.0):
        assert np.array_equal(bits(host(slayerCuda.shift(dev(x), delay, 1.0))), bits(O.shift(x, delay, 1.0)))


def test_shift_unaligned_storage_offset():
    rng = np.random.default_rng(11)
    base = dev(rng.standard_normal(2 * 3 * 64 + 1).astype(np.float32))
    x = base[1:].reshape(2, 3, 1, 1, 64)                       # 4-byte aligned only
    got = host(slayerCuda.shift(x, 5.0, 1.0))
    assert np.array_equal(got, O.shift(host(x), 5.0, 1.0))


# ------------------------------------------------------------------------------------------ conv / corr
def on_matrix_cores(op, T, Fl, generic=0):
    """Rows of whole 16-byte vectors filtered with 34..129 taps run on the matrix cores wherever the input is dense
    (the correlation always; the convolution's tiles unless they are almost all zeros, which take the event-driven
    path and keep the chain's bits).  The matrix cores add the terms in another order than the chain: those results
    are held to REL_TOL and to the element-wise bound of `close_to_chain`, all others to the chain's bits."""
    return op in ("conv", "corr") and not generic and 34 <= Fl <= 129 and T % 4 == 0 and T >= 16


def close_to_chain(got, x, f, Ts, op):
    """Element-wise bound for a sum that was added up in another order: |got - exact| <= 1e-5 * Ts * sum_i |x||f|
    (the north star's 1e-5 relative, taken against the sum of the magnitudes of each output's own terms, so a small
    output next to large ones is held as tightly as a large one).  Exact sum and bound in double precision."""
    x64, f64 = np.asarray(x, np.float64), np.asarray(f, np.float64)
    flat = x64.reshape(-1, x64.shape[-1])
    T = flat.shape[-1]
    exact, bound = np.empty_like(flat), np.empty_like(flat)
    for r in range(flat.shape[0]):
        if op == "conv":
            exact[r] = np.convolve(flat[r], f64)[:T]
            bound[r] = np.convolve(np.abs(flat[r]), np.abs(f64))[:T]
        else:
            exact[r] = np.correlate(np.concatenate([flat[r], np.zeros(len(f64) - 1)]), f64, "valid")
            bound[r] = np.correlate(np.concatenate([np.abs(flat[r]), np.zeros(len(f64) - 1)]), np.abs(f64), "valid")
    err = np.abs(np.asarray(got, np.float64).reshape(flat.shape) - exact * Ts)
    return bool(np.all(err <= 1e-5 * Ts * bound + 1e-37))


FIR_CASES = [
    # (rows shape, T, F)
    ((2, 16, 5, 5), 300, 77), ((1, 1, 1, 3), 350, 77), ((3, 70), 64, 8), ((2, 33), 2000, 8),
    ((5, 7), 100, 1), ((5, 7), 100, 2), ((5, 7), 100, 3), ((5, 7), 100, 4), ((5, 7), 100, 5),
    ((4, 9), 37, 11), ((4, 9), 40, 12), ((4, 9), 41, 13), ((3, 3), 500, 110), ((3, 3), 500, 160),
    ((2, 5), 30, 77), ((2, 2), 1, 5), ((1, 40), 700, 330), ((1, 3), 50, 500),
    # matrix-core correlation: whole rows kept as they lie in memory (T / 4 odd), padded rows, time tiles with halo,
    # fewer than 16 rows, a row count that is no multiple of 16, every window size (4..9 blocks)
    ((37,), 300, 77), ((3, 16), 304, 66), ((5,), 2000, 50), ((21,), 1000, 97), ((100,), 28, 45), ((7,), 16, 34),
    ((33,), 20, 40), ((5,), 64, 129), ((18,), 76, 113), ((40,), 44, 82), ((2, 9), 48, 34), ((1,), 300, 100),
    # whole rows of 13..16 vectors per lane, each size of the bf16 kernel's window (3..5 chunks of 32 samples)
    ((20,), 252, 120), ((17,), 204, 60), ((35,), 236, 90), ((16,), 220, 36), ((9,), 244, 100),
]


@pytest.mark.parametrize("rows,T,Fl", FIR_CASES)
@pytest.mark.parametrize("op", ["conv", "corr"])
def test_fir_matches_oracle(impl, rows, T, Fl, op):
    rng = np.random.default_rng(T * 1000 + Fl)
    x = rng.standard_normal(rows + (T,)).astype(np.float32)
    f = rng.standard_normal(Fl).astype(np.float32)
    Ts = 0.7
    got = host(getattr(slayerCuda, op)(dev(x), dev(f), Ts))
    want = getattr(O, op)(x, f, Ts, fused=True)
    assert rel_err(got, want) <= REL_TOL
    assert rel_err(got, getattr(O, op)(x, f, Ts, fused=False)) <= REL_TOL
    assert close_to_chain(got, x, f, Ts, op)
    if not on_matrix_cores(op, T, Fl, impl):
        assert np.array_equal(bits(got), bits(want)), "not bit-identical to the fused-multiply-add chain"


@pytest.mark.parametrize("Fl", [1, 5, 6, 9, 10, 13, 14, 17, 18, 25, 26, 33, 34, 49, 50, 65, 66, 77, 81, 82])
@pytest.mark.parametrize("T", [4, 12, 44, 300])
def test_fir_filter_lengths_around_kernel_choices(Fl, T):
    # the register-only kernel serves filters up to 33 taps (convolution) / 81 taps (correlation)
    # in windows of 2..22 vectors; rows whose vector count is odd end in a half-filled chunk;
    # an infinite sample must reach exactly the outputs within Fl taps of it
    rng = np.random.default_rng(Fl * 1000 + T)
    x = rng.standard_normal((3, 37, T)).astype(np.float32)
    x[1, 3, T // 2] = np.inf
    f = rng.standard_normal(Fl).astype(np.float32)
    for op in ("conv", "corr"):
        got = host(getattr(slayerCuda, op)(dev(x), dev(f), 0.5))
        want = getattr(O, op)(x, f, 0.5, fused=True)
        assert np.array_equal(np.isnan(got), np.isnan(want)), (op, Fl, T)
        if on_matrix_cores(op, T, Fl):
            # the rows that share a tile with the infinite sample are computed as chains, the others on the matrix
            # cores: the same non-finite outputs, the finite ones within the tolerance
            fin = np.isfinite(want)
            assert np.array_equal(np.isfinite(got), fin) and np.array_equal(got[~fin], want[~fin], equal_nan=True), (op, Fl, T)
            assert rel_err(np.where(fin, got, 0), np.where(fin, want, 0)) <= REL_TOL, (op, Fl, T)
        else:
            assert np.array_equal(np.where(np.isnan(got), 0, bits(got)), np.where(np.isnan(want), 0, bits(want))), (op, Fl, T)


def sum_bounds(x, f):
    """Per output of corr(x, f): the exact sum, sum |x||f| and the sum of |x| over its window, in double precision."""
    x64, f64 = np.asarray(x, np.float64), np.asarray(f, np.float64)
    pad = np.zeros(len(f64) - 1)
    exact = np.stack([np.correlate(np.concatenate([r, pad]), f64, "valid") for r in x64])
    mag = np.stack([np.correlate(np.concatenate([np.abs(r), pad]), np.abs(f64), "valid") for r in x64])
    win = np.stack([np.correlate(np.concatenate([np.abs(r), pad]), np.ones_like(f64), "valid") for r in x64])
    return exact, mag, win


@pytest.mark.parametrize("Fl", [40, 60, 77, 90, 110, 129])
def test_corr_from_split_operands_is_as_close_as_the_chain(Fl):
    # Whole rows with T / 4 odd run on bf16 matrix instructions over a three-way split of samples and taps.  The split
    # leaves out products below 2^-23 of a term and every instruction rounds its accumulator: the result stays within
    # 1e-6 of the sum of the terms' magnitudes (a tenth of the tolerance; measured: up to 4.4e-7 where one term
    # dominates a sum, 2.8e-7 on samples of one size), for samples and taps of every size and mixed signs ...
    rng = np.random.default_rng(Fl)
    T = 300
    f = (rng.standard_normal(Fl) * np.exp2(rng.integers(-20, 20, Fl))).astype(np.float32)
    for lo, hi in [(0, 1), (-60, 60), (-30, -29), (90, 100)]:
        x = (rng.standard_normal((48, T)) * np.exp2(rng.integers(lo, hi, (48, T)))).astype(np.float32)
        got = host(slayerCuda.corr(dev(x), dev(f), 1.0)).astype(np.float64)
        exact, mag, _ = sum_bounds(x, f)
        assert np.all(np.abs(got - exact) <= 1e-6 * mag), (Fl, lo, hi, np.max(np.abs(got - exact) / mag))
    # ... down to where the instruction reads a bf16 operand below 2^-126 as zero: parts of samples and taps below
    # 2^-102, at most 2^-124 * (sum |f| + sum |x| over the window) in absolute terms
    for scale in [1e-30, 1e-33, 1e-36, 1e-38, 1e-42]:
        x = (rng.standard_normal((32, T)) * scale).astype(np.float32)
        for xx, ff in [(x, f), (rng.standard_normal((32, T)).astype(np.float32), (f * np.float32(scale)).astype(np.float32))]:
            got = host(slayerCuda.corr(dev(xx), dev(ff), 1.0)).astype(np.float64)
            exact, mag, win = sum_bounds(xx, ff)
            floor = 2.0 ** -124 * (np.sum(np.abs(ff.astype(np.float64))) + win)
            assert np.all(np.abs(got - exact) <= 1e-6 * mag + floor), scale


def test_corr_from_split_operands_with_a_tap_that_is_not_finite():
    # such a tap has no split: every tile takes the chains, whose bits are the oracle's
    rng = np.random.default_rng(77)
    x = rng.standard_normal((40, 300)).astype(np.float32)
    v = (rng.standard_normal((40, 300)) * 3 + 8).astype(np.float32)
    for bad in [np.inf, -np.inf, np.nan]:
        f = rng.standard_normal(77).astype(np.float32)
        f[33] = bad
        got = host(slayerCuda.corr(dev(x), dev(f), 0.5))
        want = O.corr(x, f, 0.5, fused=True)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        assert np.array_equal(np.where(np.isnan(got), 0, bits(got)), np.where(np.isnan(want), 0, bits(want)))
        gated = host(slayerCuda.spikeBackwardCorr(dev(x), dev(v), dev(f), 10.0, 5.0, 1.0, 0.5))
        want = O.corr(O.spike_bwd(x, v, 10.0, 5.0, 1.0), f, 0.5, fused=True)
        assert np.array_equal(np.isnan(gated), np.isnan(want))
        fin = np.isfinite(want)
        assert np.array_equal(gated[~fin], want[~fin], equal_nan=True)
        assert rel_err(np.where(fin, gated, 0), np.where(fin, want, 0)) <= REL_TOL


def test_fir_sparse_spike_input_and_alpha_kernel(impl):
    rng = np.random.default_rng(5)
    x = (rng.random((4, 2, 34, 34, 300)) < 0.02).astype(np.float32)
    f = np.array(alphaKernel(10.0, 1.0, 300), dtype=np.float32)
    got = host(slayerCuda.conv(dev(x), dev(f), 1.0))
    assert np.array_equal(bits(got), bits(O.conv(x, f, 1.0)))


@pytest.mark.parametrize("T,Fl", [(300, 77), (64, 8), (300, 129), (300, 130), (350, 77), (2000, 8), (436, 9), (440, 9),
                                  (96, 1), (128, 128)])
@pytest.mark.parametrize("op", ["conv", "corr"])
def test_fir_sparse_input_edges(impl, T, Fl, op):
    # almost-all-zero rows take the event-driven path (up to 129 taps, LDS rows up to 448 samples):
    # events at both ends of a row, in neighbouring samples, negative zeros, an infinite sample
    rng = np.random.default_rng(T + Fl)
    x = np.zeros((3, 41, T), np.float32)
    x[:, :, 0] = 1.0
    x[:, :, T - 1] = -2.0
    x[0, :, T // 2: T // 2 + 3] = 0.5
    x[1, :, 1] = -0.0
    x[2, 5, T // 3] = np.inf
    idx = rng.integers(0, T, size=(3, 41, 2))
    np.put_along_axis(x, idx, rng.standard_normal((3, 41, 2)).astype(np.float32), axis=2)
    f = (rng.random(Fl) + 0.5).astype(np.float32)
    def check(x):
        got = host(getattr(slayerCuda, op)(dev(x), dev(f), 0.5))
        want = getattr(O, op)(x, f, 0.5, fused=True)
        if on_matrix_cores(op, T, Fl, impl):
            fin = np.isfinite(want)
            assert np.array_equal(np.isfinite(got), fin) and np.array_equal(got[~fin], want[~fin], equal_nan=True)
            assert rel_err(np.where(fin, got, 0), np.where(fin, want, 0)) <= REL_TOL
        else:
            assert np.array_equal(bits(got), bits(want))

    check(x)
    # the same rows with a dense row block mixed in (the choice of path is per tile)
    x[1] = rng.standard_normal((41, T)).astype(np.float32)
    check(x)


@pytest.mark.parametrize("T,Fl", [(300, 77), (304, 40), (2000, 110), (64, 129)])
def test_conv_density_switch_is_per_tile(T, Fl):
    # tiles of 16 rows choose between the event-driven path (at most one staged sample in 20 is an event; one in 40
    # when the events come in bursts) and the matrix cores: row blocks on both sides of the switch and right at it,
    # in one tensor
    rng = np.random.default_rng(T + Fl)
    f = np.array(alphaKernel(Fl / 7.7, 1.0, 2000), dtype=np.float32)[:Fl]
    f = np.concatenate([f, rng.random(Fl - len(f)).astype(np.float32)])
    blocks = []
    for pvec in (0.0, 0.05, 0.15, 0.19, 0.2, 0.21, 0.3, 1.0):       # share of non-zero vectors, one event each
        xb = np.zeros((32, T // 4, 4), np.float32)
        mask = rng.random((32, T // 4)) < pvec
        xb[mask, rng.integers(0, 4, size=int(mask.sum()))] = 1.0
        if pvec == 1.0:
            xb = rng.standard_normal(xb.shape).astype(np.float32)
        blocks.append(xb.reshape(32, T))
    for pvec in (0.004, 0.006, 0.0125, 0.05):                        # ... four events each (bursts)
        xb = np.zeros((32, T // 4, 4), np.float32)
        xb[rng.random((32, T // 4)) < pvec] = 1.0
        blocks.append(xb.reshape(32, T))
    x = np.stack(blocks)                                             # (12, 32, T)
    for op in ("conv", "corr"):
        got = host(getattr(slayerCuda, op)(dev(x), dev(f), 1.0))
        want = getattr(O, op)(x, f, 1.0, fused=True)
        assert rel_err(got, want) <= REL_TOL, op
        assert close_to_chain(got, x, f, 1.0, op), op
        if op == "conv" and T <= 448 - Fl - 16:
            # the clearly sparse blocks took the event-driven path: the chain's bits
            assert np.array_equal(bits(got[:3]), bits(want[:3]))


# ------------------------------------------------------------------------------------------ alpha kernel as a recursion
def alpha_full(tau, mult, Ts, n):
    k = np.arange(n, dtype=np.float64)
    return mult * (k * Ts / tau) * np.exp(1 - k * Ts / tau)


def close_to_alpha_sum(got, x, f, tau, mult, Ts, causal):
    """|got - exact| <= 1e-5 * Ts * sum_k |x| |h_k| element by element, h the UNTRUNCATED alpha response (the bound the
    recursion is held to; it exceeds the truncated sum's by the terms behind the window, under 1 % for gaussian or
    spike input); exact = the sum over the taps of `f` in double precision."""
    T = x.shape[-1]
    flat, out = np.asarray(x, np.float64).reshape(-1, T), np.asarray(got, np.float64).reshape(-1, T)
    h = np.abs(alpha_full(tau, mult, Ts, T + 1))
    f64 = np.asarray(f, np.float64)
    for r in range(flat.shape[0]):
        xr = flat[r] if causal else flat[r][::-1]
        yr = out[r] if causal else out[r][::-1]
        exact = np.convolve(xr, f64)[:T] * Ts
        bound = np.convolve(np.abs(xr), h)[:T] * Ts
        if np.any(np.abs(yr - exact) > 1e-5 * bound + 1e-37):
            return False
    return True


@pytest.mark.parametrize("shape,tau,mult,Ts", [((2, 6, 5, 3, 300), 10.0, 1.0, 1.0), ((1, 3, 1, 7, 64), 10.0, 1.0, 1.0),
                                               ((1, 5, 1, 1, 16), 10.0, 2.0, 1.0), ((1, 2, 1, 1, 4), 1.0, -20.0, 1.0),
                                               ((3, 9, 1, 1, 512), 20.0, 1.0, 0.5), ((1, 13, 1, 1, 352), 4.0, 1.0, 1.0),
                                               ((1, 4, 1, 1, 28), 2.0, 1.0, 1.0), ((1, 1, 1, 1, 300), 10.0, -3.0, 2.0),
                                               # rows that are not whole vectors in a tensor that is: tiles of 4 rows travel whole
                                               ((2, 6, 1, 1, 350), 10.0, 1.0, 1.0), ((1, 4, 1, 1, 33), 10.0, 1.0, 1.0),
                                               ((1, 2, 1, 1, 7), 2.0, 1.0, 1.0), ((3, 4, 1, 1, 1), 10.0, 1.0, 1.0),
                                               ((1, 10, 1, 1, 478), 25.0, 2.0, 0.5),
                                               # rows of more than 512 samples: pieces of 256 with the state carried along
                                               ((2, 5, 1, 1, 2000), 10.0, 1.0, 1.0), ((1, 6, 1, 1, 1000), 10.0, 1.0, 1.0),
                                               ((1, 3, 1, 1, 516), 4.0, 1.0, 1.0), ((1, 9, 1, 1, 1280), 10.0, -2.0, 1.0),
                                               ((1, 2, 1, 1, 4100), 30.0, 1.0, 1.0), ((1, 7, 1, 1, 772), 1.0, 1.0, 0.1),
                                               ((1, 4, 1, 1, 1028), 12.0, 1.0, 0.5)])
@pytest.mark.parametrize("kind", ["dense", "spikes"])
def test_psp_alpha_is_the_sum_over_the_taps_to_rounding(shape, tau, mult, Ts, kind):
    rng = np.random.default_rng(shape[-1] + int(tau))
    f = np.array(alphaKernel(tau, Ts, 5000, mult), dtype=np.float32)
    x = rng.standard_normal(shape).astype(np.float32) if kind == "dense" else (rng.random(shape) < 0.04).astype(np.float32)
    for causal, op in ((True, "conv"), (False, "corr")):
        got = host(slayerCuda.pspAlpha(dev(x), dev(f), tau, mult, Ts, causal))
        want = getattr(O, op)(x, f, Ts, fused=True)
        assert rel_err(got, want) <= REL_TOL, op
        assert close_to_alpha_sum(got, x, f, tau, mult, Ts, causal), op
        # ... and the adjoint identity between the two directions
    a = rng.standard_normal(shape).astype(np.float32)
    ya = host(slayerCuda.pspAlpha(dev(x), dev(f), tau, mult, Ts, True)).astype(np.float64)
    za = host(slayerCuda.pspAlpha(dev(a), dev(f), tau, mult, Ts, False)).astype(np.float64)
    lhs, rhs = float((ya * a).sum()), float((x.astype(np.float64) * za).sum())
    assert abs(lhs - rhs) <= 1e-5 * float((np.abs(ya) * np.abs(a)).sum() + 1e-30)


def test_psp_alpha_keeps_the_reach_of_a_large_sample():
    # a sample of 1e6 leaves the window after F steps: the sum over the taps is exactly zero there, the recursion's
    # difference of two running sums is zero to rounding of the untruncated terms
    tau, Ts = 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 300), dtype=np.float32)
    x = np.zeros((1, 4, 1, 1, 300), np.float32)
    x[0, 1, 0, 0, 40] = 1e6
    x[0, 2, 0, 0, 200] = -1e6
    for causal, op in ((True, "conv"), (False, "corr")):
        got = host(slayerCuda.pspAlpha(dev(x), dev(f), tau, 1.0, Ts, causal))
        want = getattr(O, op)(x, f, Ts, fused=True)
        assert close_to_alpha_sum(got, x, f, tau, 1.0, Ts, causal)
        assert rel_err(got, want) <= 1e-6
        assert np.all(got[0, 0] == 0) and np.all(got[0, 3] == 0)


@pytest.mark.parametrize("kind", ["infinity", "nan"])
def test_psp_alpha_filters_a_tile_with_a_non_finite_sample_with_the_taps(kind):
    # (a recursion would carry an infinity to the end of the row; the reference lets it reach F samples)
    rng = np.random.default_rng(9)
    tau, Ts = 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 300), dtype=np.float32)
    x = rng.standard_normal((1, 12, 1, 1, 300)).astype(np.float32)
    x[0, 5, 0, 0, 100] = np.inf if kind == "infinity" else np.nan
    for causal, op in ((True, "conv"), (False, "corr")):
        got = host(slayerCuda.pspAlpha(dev(x), dev(f), tau, 1.0, Ts, causal)).reshape(12, 300)
        want = getattr(O, op)(x, f, Ts, fused=True).reshape(12, 300)
        assert np.array_equal(bits(got[4:8]), bits(want[4:8]))      # the tile of 4 rows with the sample: the chain
        assert np.all(np.isfinite(got[:4])) and np.all(np.isfinite(got[8:]))
        assert rel_err(np.delete(got, slice(4, 8), 0), np.delete(want, slice(4, 8), 0)) <= REL_TOL


@pytest.mark.parametrize("kind", ["infinity", "nan"])
def test_psp_alpha_long_rows_switch_to_the_taps_at_a_non_finite_sample(kind):
    # rows in pieces: the pieces in front of the sample (in the direction the filter runs) are the recursion's, from
    # the sample's piece on the tile of 4 rows is the chain over the taps, bit for bit
    rng = np.random.default_rng(10)
    tau, Ts, T = 10.0, 1.0, 1200
    f = np.array(alphaKernel(tau, Ts, 300), dtype=np.float32)
    x = rng.standard_normal((1, 12, 1, 1, T)).astype(np.float32)
    x[0, 5, 0, 0, 700] = np.inf if kind == "infinity" else np.nan
    for causal, op in ((True, "conv"), (False, "corr")):
        got = host(slayerCuda.pspAlpha(dev(x), dev(f), tau, 1.0, Ts, causal)).reshape(12, T)
        want = getattr(O, op)(x, f, Ts, fused=True).reshape(12, T)
        # pieces of 256 from the end the filter starts at: the sample lies in the third one forward, the second one backward
        chain = slice(512, T) if causal else slice(0, T - 256)
        rest = slice(0, 512) if causal else slice(T - 256, T)
        assert np.array_equal(bits(got[4:8, chain]), bits(want[4:8, chain]))
        assert np.all(np.isfinite(got[4:8, rest])) and rel_err(got[4:8, rest], want[4:8, rest]) <= REL_TOL
        assert np.all(np.isfinite(got[:4])) and np.all(np.isfinite(got[8:]))
        assert rel_err(np.delete(got, slice(4, 8), 0), np.delete(want, slice(4, 8), 0)) <= REL_TOL


@pytest.mark.parametrize("shape,tau", [((1, 3, 1, 1, 350), 10.0), ((1, 2, 1, 1, 1002), 10.0), ((1, 3, 1, 1, 7), 10.0),
                                       ((1, 4, 1, 1, 1000), 40.0)])
def test_psp_alpha_outside_its_shapes_is_conv_and_corr(impl, shape, tau):
    # tensors that are not whole vectors, rows longer than 512 samples that are not whole vectors or whose kernel is
    # longer than a piece (256 taps), and forced generic kernels: the taps
    rng = np.random.default_rng(shape[-1])
    Ts = 1.0
    f = np.array(alphaKernel(tau, Ts, 1000), dtype=np.float32)
    assert tau < 40 or f.size > 256
    x = (rng.random(shape) < 0.1).astype(np.float32)
    assert torch.equal(slayerCuda.pspAlpha(dev(x), dev(f), tau, 1.0, Ts, True), slayerCuda.conv(dev(x), dev(f), Ts))
    assert torch.equal(slayerCuda.pspAlpha(dev(x), dev(f), tau, 1.0, Ts, False), slayerCuda.corr(dev(x), dev(f), Ts))


@pytest.mark.parametrize("shape,tau", [((2, 6, 5, 3, 300), 10.0), ((1, 9, 1, 1, 352), 4.0), ((3, 7, 1, 1, 64), 10.0),
                                       ((1, 1, 1, 1, 4), 1.0), ((2, 5, 1, 1, 512), 20.0), ((1, 3, 1, 1, 350), 10.0),
                                       ((1, 2, 1, 1, 1000), 10.0), ((2, 6, 1, 1, 350), 10.0), ((2, 5, 1, 1, 2000), 10.0),
                                       ((1, 3, 1, 1, 1002), 10.0)])
def test_spike_backward_psp_alpha_is_spikeBackward_then_corr(impl, shape, tau):
    # the surrogate gradient on the way in, then the correlation with the alpha kernel as a recursion: the values of
    # spikeBackward followed by pspAlpha bit for bit (the same products enter the same recursion), which is the sum over
    # the taps to rounding; shapes outside the recursion's reach run spikeBackwardCorr
    rng = np.random.default_rng(shape[-1])
    Ts, theta, tauRho, scale = 1.0, 10.0, 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 5000), dtype=np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    v = (rng.standard_normal(shape) * 4 + 8).astype(np.float32)
    got = slayerCuda.spikeBackwardPspAlpha(dev(g), dev(v), dev(f), tau, 1.0, theta, tauRho, scale, Ts)
    T = shape[-1]
    if not impl and (g.size % 4 == 0 if T <= 512 else T % 4 == 0):
        two = slayerCuda.pspAlpha(slayerCuda.spikeBackward(dev(g), dev(v), theta, tauRho, scale), dev(f), tau, 1.0, Ts, False)
        assert np.array_equal(bits(host(got)), bits(host(two)))
    else:
        assert torch.equal(got, slayerCuda.spikeBackwardCorr(dev(g), dev(v), dev(f), theta, tauRho, scale, Ts))
    gs = O.spike_bwd(g, v, theta, tauRho, scale)
    assert rel_err(host(got), O.corr(gs, f, Ts, fused=True)) <= REL_TOL
    assert close_to_alpha_sum(host(got), gs, f, tau, 1.0, Ts, False)


@pytest.mark.parametrize("shape,tau", [((2, 6, 5, 3, 300), 10.0), ((1, 9, 1, 1, 352), 4.0), ((3, 7, 1, 1, 64), 10.0),
                                       ((1, 1, 1, 1, 4), 1.0), ((2, 5, 1, 1, 512), 20.0), ((1, 3, 1, 1, 350), 10.0),
                                       ((1, 2, 1, 1, 1000), 10.0), ((2, 6, 1, 1, 350), 10.0), ((2, 5, 1, 1, 2000), 10.0),
                                       ((1, 3, 1, 1, 1002), 10.0)])
@pytest.mark.parametrize("direct", [False, True])
def test_psp_spike_backward_alpha_is_corr_then_spikeBackward(impl, shape, tau, direct):
    # the other order: the correlation with the alpha kernel as a recursion, plus the gradient that reaches the spikes
    # directly, times the surrogate gradient on the way out: the values of pspAlpha (+ add) followed by spikeBackward
    # (the same recursion; the product with the gate rounds once in both), which is the sum over the taps to rounding;
    # shapes outside the recursion's reach run corr, the addition and spikeBackward
    rng = np.random.default_rng(shape[-1] + direct)
    Ts, theta, tauRho, scale = 1.0, 10.0, 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 5000), dtype=np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    gs = rng.standard_normal(shape).astype(np.float32) if direct else None
    v = (rng.standard_normal(shape) * 4 + 8).astype(np.float32)
    got = slayerCuda.pspSpikeBackwardAlpha(dev(g), dev(gs) if direct else None, dev(v), dev(f), tau, 1.0, theta, tauRho, scale, Ts)
    T = shape[-1]
    recursion = not impl and (g.size % 4 == 0 if T <= 512 else T % 4 == 0)
    inner = slayerCuda.pspAlpha(dev(g), dev(f), tau, 1.0, Ts, False) if recursion else slayerCuda.corr(dev(g), dev(f), Ts)
    if direct:
        inner = inner + dev(gs)
    two = slayerCuda.spikeBackward(inner, dev(v), theta, tauRho, scale)
    assert np.array_equal(bits(host(got)), bits(host(two)))
    pdf = O.spike_bwd(np.ones(shape, np.float32), v, theta, tauRho, scale).astype(np.float64)
    want = (O.corr(g, f, Ts, fused=True).astype(np.float64) + (gs if direct else 0.0)) * pdf
    assert rel_err(host(got), want.astype(np.float32)) <= REL_TOL
    # element by element: the gate scales value and bound alike; the direct term adds one rounding of its own size
    T_ = shape[-1]
    h = np.abs(alpha_full(tau, 1.0, Ts, T_ + 1))
    flat_g = np.abs(g.astype(np.float64)).reshape(-1, T_)
    bound = np.stack([np.convolve(r[::-1], h)[:T_][::-1] for r in flat_g]).reshape(shape) * Ts
    if direct:
        bound = bound + np.abs(gs)
    assert np.all(np.abs(host(got) - want) <= (1e-5 * bound + 1e-37) * pdf * (1 + 1e-5) + 1e-37)


def test_psp_spike_backward_alpha_keeps_non_finite_samples_in_place():
    rng = np.random.default_rng(22)
    tau, Ts = 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 300), dtype=np.float32)
    g = rng.standard_normal((12, 300)).astype(np.float32).reshape(1, 12, 1, 1, 300)
    v = (rng.standard_normal((12, 300)) * 3 + 8).astype(np.float32).reshape(g.shape)
    g[0, 1, 0, 0, 150] = np.inf
    g[0, 10, 0, 0, 40] = np.nan
    got = slayerCuda.pspSpikeBackwardAlpha(dev(g), None, dev(v), dev(f), tau, 1.0, 10.0, 5.0, 1.0, Ts)
    # (the tiles with these samples are sums over the taps: corr, then the gate, bit for bit)
    two = slayerCuda.spikeBackward(slayerCuda.corr(dev(g), dev(f), Ts), dev(v), 10.0, 5.0, 1.0)
    gotn, twon = host(got).reshape(12, 300), host(two).reshape(12, 300)
    fin = np.isfinite(twon)
    assert not fin.all()
    assert np.array_equal(np.isfinite(gotn), fin) and np.array_equal(gotn[~fin], twon[~fin], equal_nan=True)
    assert np.array_equal(bits(gotn[0:4]), bits(twon[0:4])) and np.array_equal(bits(gotn[8:12]), bits(twon[8:12]))
    assert rel_err(np.where(fin, gotn, 0), np.where(fin, twon, 0)) <= REL_TOL


def test_spike_backward_psp_alpha_keeps_non_finite_samples_in_place():
    rng = np.random.default_rng(21)
    tau, Ts = 10.0, 1.0
    f = np.array(alphaKernel(tau, Ts, 300), dtype=np.float32)
    g = rng.standard_normal((12, 300)).astype(np.float32).reshape(1, 12, 1, 1, 300)
    v = (rng.standard_normal((12, 300)) * 3 + 8).astype(np.float32).reshape(g.shape)
    g[0, 1, 0, 0, 150] = np.inf
    v[0, 9, 0, 0, 7] = np.inf          # (gate 0 times a finite sample is 0)
    g[0, 10, 0, 0, 40] = np.nan
    got = host(slayerCuda.spikeBackwardPspAlpha(dev(g), dev(v), dev(f), tau, 1.0, 10.0, 5.0, 1.0, Ts)).reshape(12, 300)
    want = O.corr(O.spike_bwd(g, v, 10.0, 5.0, 1.0), f, Ts, fused=True).reshape(12, 300)
    fin = np.isfinite(want)
    assert not fin.all()
    assert np.array_equal(np.isfinite(got), fin) and np.array_equal(got[~fin], want[~fin], equal_nan=True)
    assert rel_err(np.where(fin, got, 0), np.where(fin, want, 0)) <= REL_TOL
    # (the tiles with these samples are sums over the taps: what the kernel that sums them gives, bit for bit)
    taps = host(slayerCuda.spikeBackwardCorr(dev(g), dev(v), dev(f), 10.0, 5.0, 1.0, Ts)).reshape(12, 300)
    assert np.array_equal(bits(got[8:12]), bits(taps[8:12]))


def test_gated_corr_on_the_matrix_cores_keeps_non_finite_samples_in_place():
    # an infinite gradient sample reaches exactly the outputs within Fl taps before it, as in the chain; so does an
    # infinite membrane potential (gate 0 times a finite sample is 0, times an infinite one NaN)
    rng = np.random.default_rng(12)
    g = rng.standard_normal((40, 300)).astype(np.float32)
    v = (rng.standard_normal((40, 300)) * 3 + 8).astype(np.float32)
    g[3, 150] = np.inf
    g[20, 7] = -np.inf
    v[20, 7] = np.inf
    f = rng.standard_normal(77).astype(np.float32)
    got = host(slayerCuda.spikeBackwardCorr(dev(g), dev(v), dev(f), 10.0, 5.0, 1.0, 0.5))
    want = O.corr(O.spike_bwd(g, v, 10.0, 5.0, 1.0), f, 0.5, fused=True)
    fin = np.isfinite(want)
    assert not fin.all()
    assert np.array_equal(np.isfinite(got), fin) and np.array_equal(got[~fin], want[~fin], equal_nan=True)
    assert rel_err(np.where(fin, got, 0), np.where(fin, want, 0)) <= REL_TOL


def test_matrix_core_corr_replayed_from_a_hip_graph():
    # the persistent matrix-core kernels (plain and gated) captured in a HIP graph: every replay, with eager work and
    # synchronisations in between, gives the bits of the eager launch
    rng = np.random.default_rng(13)
    g, v = dev(rng.standard_normal((70, 300)).astype(np.float32)), dev((rng.standard_normal((70, 300)) * 3 + 8).astype(np.float32))
    f = dev(rng.standard_normal(77).astype(np.float32))

    def both():
        return slayerCuda.corr(g, f, 1.0), slayerCuda.spikeBackwardCorr(g, v, f, 10.0, 5.0, 1.0, 1.0)

    ref = [t.clone() for t in both()]
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        both()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = both()
    for _ in range(3):
        for t in outs:
            t.fill_(-1.0)
        graph.replay()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(outs, ref))
        assert all(torch.equal(a, b) for a, b in zip(both(), ref))     # eager work between the replays
        torch.cuda.synchronize()


def test_fir_is_left_padded_conv3d(impl):
    # the identity the reference's test_slayer011 asserts: psp == pspLayer, ||diff|| / numel < 1e-6
    rng = np.random.default_rng(6)
    x = dev((rng.random((2, 4, 8, 8, 200)) < 0.1).astype(np.float32))
    f = dev(np.array(alphaKernel(10.0, 1.0, 200), dtype=np.float32))
    padded = torch.nn.functional.pad(x.reshape(2, 1, 1, -1, 200), (f.numel() - 1, 0))
    want = torch.nn.functional.conv3d(padded, torch.flip(f, [0]).reshape(1, 1, 1, 1, -1)).reshape(x.shape)
    got = slayerCuda.conv(x, f, 1.0)
    assert (torch.norm(got - want) / got.numel()).item() < 1e-6


def test_fir_adjoint_identity(impl):
    rng = np.random.default_rng(7)
    x, y = dev(rng.standard_normal((6, 50, 300)).astype(np.float32)), dev(rng.standard_normal((6, 50, 300)).astype(np.float32))
    f = dev(np.array(alphaKernel(10.0, 1.0, 300), dtype=np.float32))
    lhs = (slayerCuda.conv(x, f, 1.0).double() * y.double()).sum().item()
    rhs = (x.double() * slayerCuda.corr(y, f, 1.0).double()).sum().item()
    assert abs(lhs - rhs) <= 1e-5 * abs(lhs)


# ------------------------------------------------------------------------------------------ spike
SPIKE_CASES = [
    # (shape, nuSize)
    ((2, 16, 6, 6, 300), 11), ((1, 3, 1, 1, 350), 11), ((2, 130, 1, 1, 64), 11), ((1, 1, 1, 1, 2000), 8),
    ((3, 5, 2, 2, 95), 1), ((3, 5, 2, 2, 96), 0), ((2, 9, 3, 1, 97), 33), ((2, 9, 3, 1, 130), 34),
    ((2, 9, 3, 1, 200), 97), ((1, 70, 1, 1, 500), 110), ((1, 20, 1, 1, 501), 160), ((2, 2, 2, 2, 1), 11),
    ((1, 4, 1, 1, 7), 11),
    # rows that are not whole 16-byte vectors in tensors that are: 8-row tiles move as flat runs
    ((2, 4, 3, 1, 350), 11), ((4, 5, 1, 1, 101), 8), ((1, 8, 1, 1, 5), 3), ((1, 12, 1, 1, 351), 24),
    ((3, 4, 1, 1, 349), 16), ((1, 6, 1, 1, 101), 11),
    # rows in pieces of 512 samples: a last piece that retires more columns than a full one (488 + 32), a last
    # piece of one vector, exactly one and two pieces, a piece boundary right behind a row of 352
    ((1, 21, 1, 1, 1000), 11), ((1, 9, 1, 1, 516), 24), ((2, 5, 1, 1, 512), 11), ((1, 17, 1, 1, 1024), 16),
    ((1, 9, 1, 1, 356), 4), ((1, 3, 1, 1, 1056), 11),
]


@pytest.mark.parametrize("shape,nuSize", SPIKE_CASES)
def test_spikes_bit_exact(impl, shape, nuSize):
    rng = np.random.default_rng(shape[-1] + nuSize)
    u = (rng.standard_normal(shape) * 6).astype(np.float32)
    nu = (-rng.random(nuSize) * 12).astype(np.float32)
    if nuSize > 2:
        nu[0] = 0.0
    theta, Ts = 10.0, 0.5
    want_s, want_u = O.get_spikes(u, nu, theta, Ts)
    ud = dev(u)
    s = slayerCuda.getSpikes(ud, dev(nu), theta, Ts)
    assert np.array_equal(bits(host(s)), bits(want_s))
    assert np.array_equal(bits(host(ud)), bits(want_u)), "membrane potential must be updated in place, bit-exact"
    assert want_s.sum() > 0 or shape[-1] < 8


def test_spikes_dense_firing_and_positive_feedback(impl):
    # every sample above threshold, and a refractory kernel that pushes u up (runaway firing)
    rng = np.random.default_rng(3)
    u = (np.abs(rng.standard_normal((2, 8, 3, 3, 150))) * 5 + 10).astype(np.float32)
    for nu in (np.array([0, -1, -0.5, 3, 2], np.float32), np.array([1.0], np.float32)):
        want_s, want_u = O.get_spikes(u, nu, 10.0, 1.0)
        ud = dev(u)
        s = slayerCuda.getSpikes(ud, dev(nu), 10.0, 1.0)
        assert np.array_equal(bits(host(s)), bits(want_s)) and np.array_equal(bits(host(ud)), bits(want_u))


def test_spikes_special_cases(impl):
    rng = np.random.default_rng(4)
    u = (rng.standard_normal((1, 4, 2, 2, 90)) * 6).astype(np.float32)
    nu = np.array(alphaKernel(1.0, 1.0, 300, mult=-20), dtype=np.float32)
    ud = dev(u)
    s = slayerCuda.getSpikes(ud, dev(nu), float("inf"), 1.0)
    assert not host(s).any() and np.array_equal(host(ud), u)
    one = np.zeros((1, 1, 1, 1, 40), np.float32)
    one[..., 7] = 10.0
    od = dev(one)
    s = host(slayerCuda.getSpikes(od, dev(nu), 10.0, 0.25))
    assert s[..., 7] == 4.0 and s.sum() == 4.0
    want = one.copy()
    want[..., 7:7 + len(nu)] += nu
    assert np.array_equal(host(od), want)


# ------------------------------------------------------------------------------------------ spike backward
@pytest.mark.parametrize("n", [1, 7, 4096, 12 * 16 * 34 * 34 * 3 + 1, 1 << 20])
def test_spike_bwd(n):
    rng = np.random.default_rng(n)
    u = (rng.standard_normal(n) * 8).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    for theta, tau, scale in [(10.0, 10.0, 1.0), (10.0, 1.0, 1.0), (5120.0, 5120.0, 1 / 195.0)]:
        got = host(slayerCuda.spikeBackward(dev(g), dev(u), theta, tau, scale))
        want = O.spike_bwd(g, u, theta, tau, scale)
        np.testing.assert_allclose(got, want, rtol=REL_TOL, atol=1e-30)
        ref64 = g.astype(np.float64) * scale / tau * np.exp(-np.abs(u.astype(np.float64) - theta) / tau)
        assert rel_err(got, ref64) <= REL_TOL


@pytest.mark.parametrize("shape,Fl", [((2, 3, 5, 7, 300), 110), ((3, 41, 350), 110), ((2, 9, 64), 8), ((1, 5, 2000), 77),
                                      ((1, 2, 50), 500), ((4, 7, 1), 3),
                                      # the fused kernel on the matrix cores (rows kept as they lie in memory: T / 4 odd)
                                      ((37, 300), 77), ((3, 44), 40), ((18, 76), 113), ((100, 28), 45), ((5, 316), 129),
                                      ((19, 220), 100), ((33, 252), 60), ((40, 300), 50), ((8, 16, 300), 110)])
def test_spike_bwd_corr_is_the_two_ops_in_one(impl, shape, Fl):
    # the Loihi neuron's backward pass: pdf(voltage) * gradOut, then corr with the PSP kernel
    rng = np.random.default_rng(shape[-1] + Fl)
    v = (rng.standard_normal(shape) * 3000 + 3000).astype(np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    f = rng.random(Fl).astype(np.float32) * 100
    theta, tau, scale, Ts = 5120.0, 5120.0, 1 / 195.0, 0.5
    got = host(slayerCuda.spikeBackwardCorr(dev(g), dev(v), dev(f), theta, tau, scale, Ts))
    two = host(slayerCuda.corr(slayerCuda.spikeBackward(dev(g), dev(v), theta, tau, scale), dev(f), Ts))
    want = O.corr(O.spike_bwd(g, v, theta, tau, scale), f, Ts, fused=True)
    assert rel_err(got, want) <= REL_TOL
    assert close_to_chain(got, O.spike_bwd(g, v, theta, tau, scale), f, Ts, "corr")
    if on_matrix_cores("corr", shape[-1], Fl, impl):
        # the plain correlation of this shape runs on the matrix cores (and so does the fused kernel where the rows fit
        # its linear layout), which add the terms in another order than the chain
        assert rel_err(two, want) <= REL_TOL and rel_err(got, two) <= REL_TOL
    else:
        assert np.array_equal(bits(got), bits(two)), "fused kernel differs from spikeBackward followed by corr"


def spikes_follow_filtered_input(s, u, a, srm, nu, theta, Ts):
    """Checks (s, u) = getSpikes(psp) for SOME psp that agrees with Ts * conv(a, srm) to rounding, without knowing
    that psp's bits (a filter summed on the matrix cores): exactly, every sample without a spike ended below the
    threshold and every sample with one ended at or above fl(theta + nu[0]) - a sample is last changed when it is
    visited, and fp32 addition is monotone; and u minus the refractory responses of s is the filtered input within
    1e-5 of the sum of its terms' magnitudes (plus the rounding of the at most len(nu) additions of responses)."""
    T = a.shape[-1]
    s2, u2, a2 = (np.asarray(v).reshape(-1, T) for v in (s, u, a))
    spk = s2 != 0
    if not np.all(s2[spk] == np.float32(1.0 / Ts)):
        return False
    nu = np.asarray(nu, np.float32)
    floor = np.float32(theta) + nu[0] if len(nu) else np.float32(theta)
    if np.any(u2[~spk] >= np.float32(theta)) or np.any(u2[spk] < floor):
        return False
    f64, nu64 = np.asarray(srm, np.float64), nu.astype(np.float64)
    for r in range(a2.shape[0]):
        exact = np.convolve(a2[r].astype(np.float64), f64)[:T] * Ts
        bound = np.convolve(np.abs(a2[r]).astype(np.float64), np.abs(f64))[:T] * Ts
        refr = np.convolve(spk[r].astype(np.float64), nu64)[:T] if len(nu) else np.zeros(T)
        refr_mag = np.convolve(spk[r].astype(np.float64), np.abs(nu64))[:T] if len(nu) else np.zeros(T)
        err = np.abs(u2[r].astype(np.float64) - refr - exact)
        if np.any(err > 1e-5 * bound + 3e-6 * (np.abs(exact) + refr_mag) + 1e-37):
            return False
    return True


@pytest.mark.parametrize("shape,Fl,nuSize", [((2, 6, 5, 3, 300), 77, 11), ((1, 9, 1, 1, 352), 160, 24), ((3, 7, 1, 1, 64), 8, 4),
                                             ((1, 1, 1, 1, 4), 1, 1), ((2, 5, 1, 1, 100), 130, 16), ((1, 17, 1, 1, 8), 77, 0),
                                             ((1, 3, 1, 1, 350), 77, 11), ((1, 2, 1, 1, 2000), 8, 11), ((1, 4, 1, 1, 300), 77, 30),
                                             ((3, 11, 1, 1, 352), 129, 24), ((1, 40, 1, 1, 16), 34, 3), ((2, 9, 2, 2, 64), 50, 0),
                                             ((1, 33, 1, 1, 300), 100, 13), ((2, 16, 1, 1, 20), 40, 12)])
def test_psp_spike_is_conv_then_getSpikes(impl, shape, Fl, nuSize):
    # spike(psp(x)) in one call: what the two kernels give, on shapes that take a fused kernel (whole-vector rows up
    # to 352 samples) and on shapes that do not
    rng = np.random.default_rng(shape[-1] + Fl + nuSize)
    a = (rng.standard_normal(shape) * 2).astype(np.float32)
    srm = rng.random(Fl).astype(np.float32)
    nu = -(rng.random(nuSize) * 5).astype(np.float32)
    theta, Ts = 3.0, 0.5
    s, u = slayerCuda.pspSpike(dev(a), dev(srm), dev(nu), theta, Ts)
    u2 = slayerCuda.conv(dev(a), dev(srm), Ts)
    psp2 = host(u2).copy()
    s2 = slayerCuda.getSpikes(u2, dev(nu), theta, Ts)
    wu = O.conv(a, srm, Ts, fused=True)
    ws, wu = O.get_spikes(wu, nu, theta, Ts)
    T = shape[-1]
    one_kernel = not impl and T % 4 == 0 and T <= 352 and nuSize <= 24 and Fl <= 160
    mfma = on_matrix_cores("conv", T, Fl, impl)
    if not mfma:
        # the filter runs as the chain, fused or not: the oracle's bits
        assert np.array_equal(bits(host(s)), bits(ws)) and np.array_equal(bits(host(u)), bits(wu))
        assert torch.equal(s, s2) and np.array_equal(bits(host(u)), bits(host(u2)))
    else:
        # a dense input filtered on the matrix cores agrees with the chain to rounding; the spike function of exactly
        # those potentials follows bit for bit
        assert rel_err(psp2, O.conv(a, srm, Ts, fused=True)) <= REL_TOL
        ws2, wu2 = O.get_spikes(psp2, nu, theta, Ts)
        assert np.array_equal(bits(host(s2)), bits(ws2)) and np.array_equal(bits(host(u2)), bits(wu2))
        if one_kernel:   # the fused kernel's own potentials are not stored anywhere
            assert spikes_follow_filtered_input(host(s), host(u), a, srm, nu, theta, Ts)
            assert not spikes_follow_filtered_input(host(s), host(u) + np.float32(1e-3), a, srm, nu, theta, Ts)
            # the fused kernel and the convolution kernel sum the taps in different orders (bf16 instructions over split
            # operands here, fp32 instructions there): their potentials agree to rounding, and so do their spikes
            # except where a potential lies within that rounding of the threshold
            assert np.mean(host(s) != host(s2)) <= 1e-4
        else:
            assert torch.equal(s, s2) and np.array_equal(bits(host(u)), bits(host(u2)))
    assert ws.sum() > 0 or shape[-1] < 64


@pytest.mark.parametrize("kind", ["positive_tap", "busy_rows", "infinity", "nan", "ragged_tile"])
def test_psp_spike_on_matrix_cores_special_cases(kind):
    # the fused kernel for 34..129 taps: refractory kernels with a positive tap and rows above the threshold most of
    # the time (every sample in turn instead of candidate to candidate), non-finite samples (the tile is filtered as
    # chains: the reference's bits, infinities and NaNs where the reference puts them), a last tile of 3 rows
    rng = np.random.default_rng(len(kind))
    shape = (2, 19, 1, 1, 300) if kind == "ragged_tile" else (2, 24, 1, 1, 300)
    a = (rng.standard_normal(shape) * 2).astype(np.float32)
    srm = (rng.random(77).astype(np.float32) - 0.3)
    nu = -(rng.random(11) * 5).astype(np.float32)
    theta, Ts = 3.0, 1.0
    if kind == "positive_tap":
        nu[4] = 1.5
    if kind == "busy_rows":
        theta = -2.0
    if kind == "infinity":
        a[0, 3, 0, 0, 100] = np.inf
        a[1, 20, 0, 0, 299] = -np.inf
    if kind == "nan":
        a[1, 7, 0, 0, 0] = np.nan
    s, u = slayerCuda.pspSpike(dev(a), dev(srm), dev(nu), theta, Ts)
    s, u = host(s), host(u)
    flat_a, flat_s, flat_u = a.reshape(-1, 300), s.reshape(-1, 300), u.reshape(-1, 300)
    chain_u = O.conv(a, srm, Ts, fused=True)
    chain_s, chain_u = O.get_spikes(chain_u, nu, theta, Ts)
    chain_s, chain_u = chain_s.reshape(-1, 300), chain_u.reshape(-1, 300)
    for tile in range(0, flat_a.shape[0], 16):
        rows = slice(tile, tile + 16)
        if not np.all(np.isfinite(flat_a[rows])):
            assert np.array_equal(bits(flat_s[rows]), bits(chain_s[rows]))
            assert np.array_equal(bits(flat_u[rows]), bits(chain_u[rows]))
        elif kind == "positive_tap":
            # rows whose spikes are the chain's (a potential within rounding of the threshold may flip one) end at the
            # chain's potentials to rounding
            same = [r for r in range(tile, min(tile + 16, flat_a.shape[0])) if np.array_equal(flat_s[r], chain_s[r])]
            assert len(same) >= 12
            for r in same:
                assert np.max(np.abs(flat_u[r].astype(np.float64) - chain_u[r])) <= 1e-5 * np.max(np.abs(chain_u[r]))
        else:
            assert spikes_follow_filtered_input(flat_s[rows], flat_u[rows], flat_a[rows], srm, nu, theta, Ts)
    u2 = slayerCuda.conv(dev(a), dev(srm), Ts)
    s2 = slayerCuda.getSpikes(u2, dev(nu), theta, Ts)
    if kind in ("positive_tap", "busy_rows", "ragged_tile"):
        # the two kernels sum the taps in another order than the fused one: the same spikes except where a potential
        # lies within rounding of the threshold, and the same potentials to rounding in the rows with the same spikes
        s2, u2 = host(s2).reshape(-1, 300), host(u2).reshape(-1, 300)
        same = [r for r in range(flat_s.shape[0]) if np.array_equal(flat_s[r], s2[r])]
        assert len(same) >= 0.9 * flat_s.shape[0]
        for r in same:
            assert np.max(np.abs(flat_u[r].astype(np.float64) - u2[r])) <= 1e-5 * np.max(np.abs(u2[r]))
    assert flat_s.sum() > 0


def test_spikes_many_long_rows_use_16_row_tiles():
    # enough long rows to fill the GPU with 16-row tiles (pieces of 256 samples): sampled rows against the oracle
    rng = np.random.default_rng(77)
    rows, T = 70000, 400
    u = (rng.standard_normal((1, rows, 1, 1, T)) * 6).astype(np.float32)
    nu = np.array(alphaKernel(1.0, 1.0, T, mult=-20.0), dtype=np.float32)
    ud = dev(u)
    s = host(slayerCuda.getSpikes(ud, dev(nu), 10.0, 1.0)).reshape(rows, T)
    un = host(ud).reshape(rows, T)
    pick = np.concatenate([np.arange(40), rng.integers(0, rows, 400), np.arange(rows - 40, rows)])
    ws, wu = O.get_spikes(u.reshape(rows, T)[pick].reshape(1, len(pick), 1, 1, T), nu, 10.0, 1.0)
    assert np.array_equal(bits(s[pick]), bits(ws.reshape(len(pick), T)))
    assert np.array_equal(bits(un[pick]), bits(wu.reshape(len(pick), T)))
    assert ws.sum() > 0


# ------------------------------------------------------------------------------------------ delay gradient
@pytest.mark.parametrize("shape,Ts", [((4, 6, 1, 1, 80), 0.1), ((64, 20, 1, 1, 2000), 1.0), ((3, 2, 5, 7, 33), 0.5),
                                      ((1, 1, 1, 1, 1), 1.0)])
def test_delay_grad(shape, Ts):
    rng = np.random.default_rng(shape[-1])
    y = rng.standard_normal(shape).astype(np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    got = host(slayerCuda.delayGrad(dev(y), dev(g), Ts))
    want = O.delay_grad(y, g, Ts)
    assert got.shape == shape[1:-1]
    assert rel_err(got, want) <= REL_TOL
    # the three-pass formulation of the reference: conv with [-1, 1]/Ts (Ts argument 1), multiply, sum
    diff = slayerCuda.conv(dev(y), dev(np.array([-1, 1], np.float32)) / Ts, 1)
    ref = torch.sum(dev(g).double() * diff.double(), [0, -1]) * Ts
    assert rel_err(got, host(ref)) <= REL_TOL


# ------------------------------------------------------------------------------------------ Loihi
def loihi_input(rng, shape, p=0.05):
    return (2 * rng.integers(-128, 128, size=shape) * (rng.random(shape) < p)).astype(np.float32)


@pytest.mark.parametrize("shape", [(2, 16, 8, 8, 300), (1, 3, 1, 1, 350), (2, 130, 1, 1, 64), (64, 200), (5, 1),
                                   (1, 1, 1, 1, 2000), (70, 33)])
@pytest.mark.parametrize("refDelay", [1, 2, 17])
def test_loihi_bit_exact(impl, shape, refDelay):
    rng = np.random.default_rng(sum(shape) + refDelay)
    w = loihi_input(rng, shape, p=0.3)
    want = O.loihi_get_spikes(w, 0, 80 * 64, 1024, 128, refDelay)
    got = slayerLoihiCuda.getSpikes(dev(w), 0, 80 * 64, 1024, 128, refDelay)
    for a, b, name in zip(got, want, ("spike", "voltage", "current")):
        assert np.array_equal(bits(host(a)), bits(b)), name
    assert want[0].sum() > 0 or shape[-1] < 8


@pytest.mark.parametrize("shape", [(2, 16, 8, 8, 300), (3, 41, 64), (1, 3, 1, 1, 350), (2, 70, 96), (5, 1), (9, 33),
                                   (1, 2, 2000), (64, 40)])
@pytest.mark.parametrize("delay", [0, 1, 5, 31])
def test_loihi_delayed_spikes_and_optional_outputs(impl, shape, delay):
    # the fused form is getSpikes followed by a shift of the spike tensor by `delay` samples;
    # voltage and current are not shifted and may be left out
    rng = np.random.default_rng(sum(shape) + delay)
    w = loihi_input(rng, shape, p=0.3)
    ws, wv, wu = O.loihi_get_spikes(w, 0, 80 * 64, 1024, 128, 2)
    want_s = O.shift(ws, float(delay), 1.0)
    s, v, u = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 80 * 64, 1024, 128, 2, delay)
    assert np.array_equal(bits(host(s)), bits(want_s)), "spike"
    assert np.array_equal(bits(host(v)), bits(wv)), "voltage"
    assert np.array_equal(bits(host(u)), bits(wu)), "current"
    s2, v2, u2 = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 80 * 64, 1024, 128, 2, delay, voltage=True, current=False)
    assert u2 is None and np.array_equal(host(s2), want_s) and np.array_equal(host(v2), wv)
    s3, v3, u3 = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 80 * 64, 1024, 128, 2, delay, voltage=False, current=False)
    assert v3 is None and u3 is None and np.array_equal(host(s3), want_s)
    # and it is what the two separate calls give
    two = slayerCuda.shift(slayerLoihiCuda.getSpikes(dev(w), 0, 80 * 64, 1024, 128, 2)[0], float(delay), 1.0)
    assert torch.equal(s, two)


@pytest.mark.parametrize("step", [2, 1, 0.5, 0.3, 3.0, -2.0, 1e-3])
def test_loihi_weight_quantiser_is_the_tensor_expression(step):
    # round(w / step) * step as one kernel: bit for bit what torch makes of the expression on the GPU, ties included
    rng = np.random.default_rng(3)
    w = (rng.standard_normal((7, 5, 3, 3, 1)) * 9).astype(np.float32)
    w.reshape(-1)[:12] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, 3.0, -3.0, 0.0, -0.0, 1.0, 1e9, -1e-9], np.float32) * step
    wt = dev(w)
    got = slayerLoihiCuda.quantize(wt, step)
    want = torch.round(wt / step) * step
    assert np.array_equal(bits(host(got)), bits(host(want)))
    from slayerpytorch_amd import slayerLoihi
    x = dev(w).requires_grad_(True)
    y = slayerLoihi.quantize(x, step)
    assert np.array_equal(bits(host(y)), bits(host(want)))
    y.backward(torch.ones_like(y))
    assert torch.equal(x.grad, torch.ones_like(x))           # straight-through gradient
    assert slayerLoihiCuda.quantize(torch.zeros((0,), device="cuda"), 2).numel() == 0
    with pytest.raises(ValueError):
        slayerLoihiCuda.quantize(wt, 0)


def test_loihi_delay_limits():
    w = dev(np.zeros((2, 3, 40), np.float32))
    with pytest.raises(ValueError):
        slayerLoihiCuda.getSpikesDelayed(w, 0, 5120, 1024, 128, 1, 32)
    with pytest.raises(TypeError):
        slayerLoihiCuda.getSpikesDelayed(w, 0, 5120, 1024, 128, 1, -1)
    lib = _lib.load()
    assert lib.slayer_loihi_get_spikes_delayed_f32(None, None, None, None, 4, 8, 0, 5120, 1024, 128, 1, 32, None) == 2
    assert lib.slayer_loihi_get_spikes_delayed_f32(None, None, None, None, 4, 8, 0, 5120, 1024, 128, 1, -1, None) == 1


@pytest.mark.parametrize("params", [(1, 10 * 64, 2048, 256, 3), (0, 64, 0, 0, 1), (2, 5000, 4095, 4095, 2),
                                    (0, 1, 4096, 4096, 1), (3, 300000, 100, 10, 500)])
def test_loihi_parameters_wraparound_and_truncation(impl, params):
    rng = np.random.default_rng(8)
    w = (rng.standard_normal((3, 40, 150)) * 40).astype(np.float32)           # non-integers: (int) truncates toward zero
    w[0, 0, 5] = np.nan
    w[0, 1, 5] = 1e20
    w[0, 2, 5] = -1e20
    want = O.loihi_get_spikes(w, *params)
    got = slayerLoihiCuda.getSpikes(dev(w), *params)
    for a, b, name in zip(got, want, ("spike", "voltage", "current")):
        assert np.array_equal(bits(host(a)), bits(b)), name


@pytest.mark.parametrize("scale", [1, 6, 30, 200])
@pytest.mark.parametrize("params", [(0, 80 * 64, 1024, 128, 2), (2, 3000 * 64, 64, 16, 1), (3, 100000 * 64, 0, 0, 3),
                                    (1, 5000, 4096, 4096, 1), (0, 5000, 5000, 4097, 1)])
def test_loihi_states_around_the_range_of_the_short_multiplication(impl, scale, params):
    # the kernel multiplies with 24-bit operands while current and voltage stay below 2^19 in magnitude and
    # falls back to the 32-bit wrap-around arithmetic for the 32 samples in which either leaves that range:
    # inputs scaled so that rows stay inside, cross the limit in both directions, or live far outside it
    rng = np.random.default_rng(scale + params[0])
    w = (loihi_input(rng, (3, 50, 300), p=0.3) * scale).astype(np.float32)
    w[1] = np.abs(w[1])                                  # monotonic rows reach the limit soonest
    w[2, :25] = -np.abs(w[2, :25])
    want = O.loihi_get_spikes(w, *params)
    assert max(np.abs(want[1]).max(), np.abs(want[2]).max()) > 2 ** 19 or scale <= 6
    got = slayerLoihiCuda.getSpikes(dev(w), *params)
    for a, b, name in zip(got, want, ("spike", "voltage", "current")):
        assert np.array_equal(bits(host(a)), bits(b)), name
    s2, v2, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), *params, 0, voltage=True, current=False)
    assert np.array_equal(bits(host(s2)), bits(want[0])) and np.array_equal(bits(host(v2)), bits(want[1]))
    s3, _, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), *params, 1, voltage=False, current=False)
    assert np.array_equal(bits(host(s3)), bits(O.shift(want[0], 1.0, 1.0)))


@pytest.mark.parametrize("T", [64, 68, 72, 100, 124, 128, 132, 196, 300, 332])
@pytest.mark.parametrize("rows", [(1, 1), (3, 67), (2, 64), (5, 13)])
def test_loihi_rows_sharing_memory_lines(impl, T, rows):
    # rows that are whole 16-byte vectors but start and end inside 128-byte memory lines: the line
    # shared by two neighbouring rows is written once, from the results of both
    rng = np.random.default_rng(T)
    w = loihi_input(rng, rows + (T,), p=0.3)
    want = O.loihi_get_spikes(w, 0, 20 * 64, 1024, 128, 2)
    got = slayerLoihiCuda.getSpikes(dev(w), 0, 20 * 64, 1024, 128, 2)
    for a, b, name in zip(got, want, ("spike", "voltage", "current")):
        assert np.array_equal(bits(host(a)), bits(b)), name
    assert want[0].sum() > 0
    # without the current among the outputs a tile is 64 rows
    s2, v2, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 20 * 64, 1024, 128, 2, 0, voltage=True, current=False)
    assert np.array_equal(bits(host(s2)), bits(want[0])) and np.array_equal(bits(host(v2)), bits(want[1]))
    s3, _, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 20 * 64, 1024, 128, 2, 2, voltage=False, current=False)
    assert np.array_equal(bits(host(s3)), bits(O.shift(want[0], 2.0, 1.0)))


@pytest.mark.parametrize("T", [65, 66, 67, 95, 97, 101, 127, 129, 350, 351, 2001])
@pytest.mark.parametrize("rows", [(4, 1), (4, 33), (8, 8), (2, 2, 3, 5), (12, 3), (4, 67)])
@pytest.mark.parametrize("delay", [0, 3])
def test_loihi_rows_that_are_not_whole_vectors(impl, T, rows, delay):
    # T % 4 != 0 in a tensor of whole vectors: the 16-byte vector in which a row ends also holds the
    # first samples of the next row; tiles of 32 or 64 rows still begin and end on memory lines
    rng = np.random.default_rng(T + len(rows))
    w = loihi_input(rng, rows + (T,), p=0.3)
    ws, wv, wu = O.loihi_get_spikes(w, 0, 20 * 64, 1024, 128, 2)
    s, v, u = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 20 * 64, 1024, 128, 2, delay)
    assert np.array_equal(bits(host(s)), bits(O.shift(ws, float(delay), 1.0))), "spike"
    assert np.array_equal(bits(host(v)), bits(wv)), "voltage"
    assert np.array_equal(bits(host(u)), bits(wu)), "current"
    assert ws.sum() > 0
    # without the current among the outputs a tile is 64 rows
    s2, v2, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 20 * 64, 1024, 128, 2, delay, voltage=True, current=False)
    assert np.array_equal(bits(host(s2)), bits(host(s))) and np.array_equal(bits(host(v2)), bits(wv))
    s3, _, _ = slayerLoihiCuda.getSpikesDelayed(dev(w), 0, 20 * 64, 1024, 128, 2, delay, voltage=False, current=False)
    assert np.array_equal(bits(host(s3)), bits(host(s)))


def test_loihi_unaligned_tensors_take_the_general_kernel():
    rng = np.random.default_rng(77)
    w = loihi_input(rng, (2 * 40 * 96 + 1,), p=0.3)
    wt = dev(w)[1:].reshape(2, 40, 96)                       # 4-byte aligned storage only
    want = O.loihi_get_spikes(w[1:].reshape(2, 40, 96), 0, 20 * 64, 1024, 128, 1)
    got = slayerLoihiCuda.getSpikes(wt, 0, 20 * 64, 1024, 128, 1)
    for a, b in zip(got, want):
        assert np.array_equal(host(a), b)


# ------------------------------------------------------------------------------------------ empty tensors
def test_empty_tensors():
    e = torch.empty((0, 3, 1, 1, 10), device="cuda")
    f = dev(np.ones(3, np.float32))
    assert slayerCuda.conv(e, f, 1.0).shape == e.shape
    assert slayerCuda.corr(e, f, 1.0).shape == e.shape
    assert slayerCuda.shift(e, 2.0).shape == e.shape
    assert slayerCuda.getSpikes(e, f, 1.0, 1.0).shape == e.shape
    assert [t.shape for t in slayerLoihiCuda.getSpikes(e, 0, 64, 0, 0, 1)] == [e.shape] * 3
    z = torch.empty((2, 3, 1, 1, 0), device="cuda")
    assert slayerCuda.conv(z, f, 1.0).shape == z.shape
    assert slayerCuda.getSpikes(z, f, 1.0, 1.0).shape == z.shape
    assert host(slayerCuda.delayGrad(z, z, 1.0)).tolist() == [[[0.0]]] * 3
    torch.cuda.synchronize()


# ------------------------------------------------------------------ spike with the shift fused in
@pytest.mark.parametrize("shape", [(3, 5, 4, 4, 300), (2, 3, 2, 2, 352), (2, 7, 1, 1, 100), (2, 3, 1, 1, 7),
                                   (4, 3, 2, 2, 350), (1, 9, 1, 1, 33), (2, 4, 1, 1, 2000), (3, 21, 1, 1, 1000),
                                   (1, 9, 1, 1, 356), (2, 40, 1, 1, 512), (1, 3, 1, 1, 2002)])
@pytest.mark.parametrize("delay", ["scalar", "negative", "zero", "huge", "table", "one-element", "far", "far-negative",
                                   "long-table"])
def test_spike_delayed_equals_spike_then_shift(shape, delay, impl):
    """getSpikesDelayed against the two kernels it fuses (both already pinned to the oracle), and
    against the oracle itself: bit-exact, membrane potential included.  Rows longer than 352 samples travel in
    pieces: the fused kernel keeps their spike bits and stores the shifted spikes after the last piece, for
    shifts of any size and sign ("far": beyond a piece).  (1, 3, 1, 1, 2002) and the generic kernels are shapes
    the fused kernel declines: the wrapper then runs the two kernels."""
    rng = np.random.default_rng(31)
    Ts, dTs = 1.0, 0.5
    u = (rng.standard_normal(shape) * 6 + 4).astype(np.float32)
    nu = np.array(alphaKernel(1.0, Ts, shape[-1], mult=-20.0), dtype=np.float32)
    d = {"scalar": 3.4, "negative": -2.6, "zero": 0.0, "huge": 1e9, "far": 300.3, "far-negative": -170.0,
         "table": (rng.random(shape[1:4]) * 12 - 2).astype(np.float32),
         "long-table": ((rng.random(shape[1:4]) * 2 - 1) * shape[-1] * 0.3).astype(np.float32),
         "one-element": np.array([5.0], dtype=np.float32)}[delay]
    dd = dev(d) if isinstance(d, np.ndarray) else d
    ua, ub = dev(u), dev(u)
    got = slayerCuda.getSpikesDelayed(ua, dev(nu), 10.0, Ts, dd, dTs)
    ref = slayerCuda.shift(slayerCuda.getSpikes(ub, dev(nu), 10.0, Ts), dd, dTs)
    assert np.array_equal(bits(host(got)), bits(host(ref)))
    assert np.array_equal(bits(host(ua)), bits(host(ub)))
    s_ref, u_ref = O.get_spikes(u, nu, 10.0, Ts)
    assert np.array_equal(bits(host(got)), bits(O.shift(s_ref, d, dTs)))
    assert np.array_equal(bits(host(ua)), bits(u_ref))
    assert s_ref.sum() > 0


@pytest.mark.parametrize("shape", [(3, 5, 4, 4, 300), (2, 3, 1, 1, 7), (4, 3, 2, 2, 350), (2, 4, 1, 1, 2000)])
@pytest.mark.parametrize("delay", ["scalar", "negative", "huge", "table"])
def test_spike_backward_delayed_equals_shift_then_spike_backward(shape, delay):
    rng = np.random.default_rng(32)
    dTs = 0.5
    u = (rng.standard_normal(shape) * 6 + 4).astype(np.float32)
    g = rng.standard_normal(shape).astype(np.float32)
    d = {"scalar": 3.4, "negative": -2.6, "huge": 1e9,
         "table": (rng.random(shape[1:4]) * 12 - 2).astype(np.float32)}[delay]
    dd = dev(d) if isinstance(d, np.ndarray) else d
    got = slayerCuda.spikeBackwardDelayed(dev(g), dev(u), 10.0, 10.0, 1.0, dd, dTs)
    ref = slayerCuda.spikeBackward(slayerCuda.shift(dev(g), dd, dTs, sign=-1.0), dev(u), 10.0, 10.0, 1.0)
    assert np.array_equal(bits(host(got)), bits(host(ref)))
    neg = -d if isinstance(d, np.ndarray) else -d
    want = O.spike_bwd(O.shift(g, neg, dTs), u, 10.0, 10.0, 1.0)
    assert rel_err(host(got), want) <= REL_TOL

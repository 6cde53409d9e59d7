"""The entry point that allocates nothing, ``slayer_delay_grad_static_f32``, against the entry point it is a
variant of, ``slayer_delay_grad_f32``: both are called through the C ABI (ctypes) on the same device buffers
and must agree bit for bit (same kernels, same fixed summation order; only the home of the partial sums
differs), on two calls in a row, the second with a smaller input - the library's array then still holds the
first call's partial sums.  Every tensor is allocated before the first call.
"""
import numpy as np
import pytest
import torch

from oracle import oracle as O
from slayerpytorch_amd import _lib

from _util import rel_err

pytestmark = pytest.mark.gpu


def _call(lib, entry, gradDelay, y, g, workspace, shape, Ts, stream):
    nBatch, T = shape[0], shape[-1]
    nPerBatch = int(np.prod(shape[1:-1]))
    if workspace is None:
        return getattr(lib, entry)(gradDelay.data_ptr(), y.data_ptr(), g.data_ptr(), nBatch, nPerBatch, T, Ts, stream)
    return getattr(lib, entry)(gradDelay.data_ptr(), y.data_ptr(), g.data_ptr(), workspace.data_ptr(), nBatch,
                               nPerBatch, T, Ts, stream)


def test_static_delay_gradient_matches_workspace_entry_point():
    lib = _lib.load()
    rng = np.random.default_rng(77)
    shapes = [(64, 256, 1, 1, 2000), (5, 3, 7, 2, 132), (3, 2, 5, 1, 33)]  # the second and third are smaller
    Ts = 0.5
    cases = []
    for shape in shapes:
        y = rng.standard_normal(shape).astype(np.float32)
        g = rng.standard_normal(shape).astype(np.float32)
        rows = int(np.prod(shape[:-1]))
        assert rows <= lib.slayer_delay_grad_static_max_rows()
        cases.append((shape, y, g, torch.from_numpy(y).cuda(), torch.from_numpy(g).cuda(),
                      torch.full(shape[1:-1], np.nan, dtype=torch.float32, device="cuda"),
                      torch.full(shape[1:-1], np.nan, dtype=torch.float32, device="cuda"),
                      torch.empty(rows, dtype=torch.float32, device="cuda")))
    stream = torch.cuda.current_stream().cuda_stream
    # a first call on this device looks up the array's address (once per device); what is checked below is that the
    # calls after it take no memory from the device - the free bytes the driver reports, which also sees an allocation
    # made inside the library, and torch's own count
    shape0, _, _, dy0, dg0, got0, _, _ = cases[-1]
    assert _call(lib, "slayer_delay_grad_static_f32", got0, dy0, dg0, None, shape0, Ts, stream) == 0
    torch.cuda.synchronize()
    before, freeBefore = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
    for shape, y, g, dy, dg, gotStatic, gotWorkspace, workspace in cases:   # back to back, no sync in between
        assert _call(lib, "slayer_delay_grad_static_f32", gotStatic, dy, dg, None, shape, Ts, stream) == 0
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before and torch.cuda.mem_get_info()[0] == freeBefore
    for shape, y, g, dy, dg, gotStatic, gotWorkspace, workspace in cases:
        assert _call(lib, "slayer_delay_grad_f32", gotWorkspace, dy, dg, workspace, shape, Ts, stream) == 0
    torch.cuda.synchronize()
    for shape, y, g, dy, dg, gotStatic, gotWorkspace, workspace in cases:
        a, b = gotStatic.cpu().numpy(), gotWorkspace.cpu().numpy()
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), shape
        assert rel_err(a, O.delay_grad(y, g, Ts)) <= 1e-5, shape


def test_static_delay_gradient_rejects_sizes_beyond_its_array():
    lib = _lib.load()
    limit = lib.slayer_delay_grad_static_max_rows()
    tiny = torch.zeros(8, device="cuda")
    # nothing is launched for a rejected size, so the pointers are never used
    assert lib.slayer_delay_grad_static_f32(tiny.data_ptr(), tiny.data_ptr(), tiny.data_ptr(), limit + 1, 1, 4, 1.0,
                                            None) == 2
    assert lib.slayer_delay_grad_static_f32(tiny.data_ptr(), tiny.data_ptr(), tiny.data_ptr(), 1 << 40, 1 << 40, 4,
                                            1.0, None) == 2
    assert lib.slayer_delay_grad_static_f32(tiny.data_ptr(), tiny.data_ptr(), tiny.data_ptr(), -1, 1, 4, 1.0,
                                            None) == 1
    torch.cuda.synchronize()

"""Helpers around the layer engines that the reference has no counterpart for.

``capturedStep``: a training or inference step recorded once in a HIP graph and replayed.  The kernels of this
package only enqueue work on the stream they are given - no allocation of their own, no host synchronisation -
so a whole step (synapses, psp, spike, delays, loss, backward, optimiser) can be captured; a step of many short
launches then costs one graph launch instead of one launch per kernel.
"""
import torch


class capturedStep:
    """``step = capturedStep(fn)``; ``out = step()`` runs ``fn()`` from a HIP graph.

    ``fn`` takes no arguments: it reads its batch from tensors that stay the same objects between calls (copy
    each new batch into them with ``copy_``) and returns a tensor, a tuple / list of tensors or None.  The first
    call runs ``fn`` ``warmup`` times on a side stream (lazy initialisation, the caching allocator's pools, the
    parameters' ``.grad`` tensors), records it once, and replays the recording; later calls only replay.  What
    ``fn`` returned during recording is returned by every call: the same tensors, overwritten by each replay.

    Rules for ``fn``, as for any captured PyTorch code: no host reads of device values (``.item()``, ``print`` of
    a tensor, a Python branch on one), gradients zeroed in place (``optimizer.zero_grad(set_to_none=False)`` or
    ``p.grad.zero_()``), an optimiser built with ``capturable=True`` if it steps inside.  The dense layer's
    event-driven kernels are chosen from the density measured during the warm-up calls, which therefore have to
    see a representative batch.
    """

    def __init__(self, fn, warmup=3, pool=None):
        if warmup < 1:
            raise ValueError("capturedStep needs at least one warm-up call before recording")
        self.fn = fn
        self.warmup = int(warmup)
        self.pool = pool
        self.graph = None
        self.result = None

    def capture(self):
        """Warm up and record now (otherwise done by the first call)."""
        if not torch.cuda.is_available():
            raise RuntimeError("capturedStep needs a GPU")
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(self.warmup):
                self.fn()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, pool=self.pool):
            self.result = self.fn()
        self.graph = graph
        return self

    def __call__(self):
        if self.graph is None:
            self.capture()
        self.graph.replay()
        return self.result

    def reset(self):
        """Drops the recording (after a change of shapes, layers or switches); the next call records again."""
        self.graph = None
        self.result = None

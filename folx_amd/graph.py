"""``jit``: replay a forward-Laplacian evaluation as one captured HIP graph.

The reference wraps ``forward_laplacian`` in ``jax.jit`` (folx/interpreter.py:352): the
Python interpreter runs once per input shape and later calls launch the compiled
executable.  The equivalent here is stream capture: the first call for an input shape
runs eagerly (it fills the device caches of index tables and constants), the second is
captured into a HIP graph together with all its allocations, and every later call copies
the input into the graph's static buffer and replays it -- no Python rule code, no host
index algebra, one launch.

Only fill kernels are used to clear memory inside the rules (never memset nodes), and no
host-to-device copy happens once the caches are warm, so the captured region contains
nothing but kernel nodes and device-to-device copies.
"""

from __future__ import annotations

import gc

import torch

from .api import BatchedArray, FwdJacobian, FwdLaplArray


def _flatten(out):
    """-> (list of tensors, rebuild(list of tensors))"""
    if isinstance(out, torch.Tensor):
        return [out], lambda ts: ts[0]
    if isinstance(out, BatchedArray):
        return [out.data], lambda ts: BatchedArray(ts[0])
    if isinstance(out, FwdLaplArray):
        mask = out.jacobian.x0_idx
        return ([out.x, out.jacobian.data, out.laplacian],
                lambda ts: FwdLaplArray(ts[0], FwdJacobian(ts[1], mask), ts[2]))
    if isinstance(out, (tuple, list)):
        parts = [_flatten(o) for o in out]
        sizes = [len(p[0]) for p in parts]
        tensors = [t for p in parts for t in p[0]]

        def rebuild(ts):
            res, i = [], 0
            for (_, rb), n in zip(parts, sizes):
                res.append(rb(ts[i : i + n]))
                i += n
            return type(out)(res)

        return tensors, rebuild
    raise TypeError(f'cannot capture an output of type {type(out)}')


class _Captured:
    def __init__(self, fn, x):
        self.static_in = x.clone()
        # warm-up on a side stream (allocator and caches reach their steady state)
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            fn(self.static_in)
        torch.cuda.current_stream().wait_stream(s)
        torch.cuda.synchronize()
        self.graph = torch.cuda.CUDAGraph()
        # No finalizer may run while the capture is open: a dead reference cycle that still owns
        # an older graph (or its memory pool) would destroy it through HIP calls that are not
        # allowed during a capture and end the process.  Such cycles are collected now, and the
        # collector stays off until the capture is closed (torch.cuda.graph itself no longer
        # collects before capturing).
        gc.collect()
        gc_on = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(self.graph):
                out = fn(self.static_in)
        finally:
            if gc_on:
                gc.enable()
        self.tensors, self.rebuild = _flatten(out)
        # the graph reads the cached index tables and constants by address: they stay alive with it,
        # whatever the caches drop later
        from . import sparse_ops

        self._keepalive = sparse_ops.cached_tensors()

    def __call__(self, x):
        self.static_in.copy_(x)
        self.graph.replay()
        # results live in the graph's memory pool and are overwritten by the next replay
        return self.rebuild([t.clone() for t in self.tensors])


class _Jitted:
    """Callable returned by ``jit``; an object rather than a function carrying itself as an
    attribute, so that dropping it frees its graphs at once (no reference cycle)."""

    def __init__(self, fn):
        self.eager = fn
        self._captured: dict = {}
        self._seen: set = set()

    def __call__(self, x):
        if not isinstance(x, torch.Tensor):
            x = torch.as_tensor(x, dtype=torch.float32)
        x = x.to(device='cuda', dtype=torch.float32).contiguous()
        key = tuple(x.shape)
        if key in self._captured:
            return self._captured[key](x)
        if key not in self._seen:
            self._seen.add(key)
            return self.eager(x)
        self._captured[key] = _Captured(self.eager, x)
        return self._captured[key](x)

    def batched(self, x):
        return self(x)

    def invalidate(self):
        """Drop the captured graphs: the next calls run eagerly and capture again.  Needed after
        anything the function closes over has been REPLACED -- a weight rebound to a new tensor, a
        numpy weight or constant changed (those are baked in by content at capture), another
        sparsity threshold.  Device tensors updated IN PLACE need nothing: the graph reads them by
        address."""
        self._captured.clear()
        self._seen.clear()


def jit(fn):
    """Wrap ``fn(x) -> FwdLaplArray | tensors`` (``x`` a device tensor with the walker axis
    first, e.g. ``vmap(forward_laplacian(f, thr))``) so that repeated calls with the same
    input shape replay one HIP graph.  The first call per shape runs eagerly.

    Unlike ``jax.jit``, which takes parameters as traced arguments, the graph bakes in whatever
    ``fn`` closes over: device tensors by address (update them in place, e.g. ``w.copy_(new)``,
    and replays see the new values), numpy arrays by their content at capture time.  After
    rebinding a weight to another tensor or changing a numpy weight call ``.invalidate()`` on the
    returned object."""
    return _Jitted(fn)

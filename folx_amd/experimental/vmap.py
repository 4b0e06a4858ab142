"""``auto_batched_vmap`` (folx/experimental/vmap.py:14-73): ``batched_vmap`` with the chunk size taken from a
measurement of the function's memory use instead of from the caller.

The reference compares the compiled memory of one and of two samples; here the function is RUN on two small
chunks of the caller's own batch and the allocator's peak is read after each (``torch.cuda.max_memory_allocated``),
which also counts the workspaces of the HIP entry points and the constants that are uploaded once.  From
``peak(n) = base + n * per_walker`` the largest chunk that fits ``max_fraction`` of the memory that is free now
follows.  The probes cost two small evaluations on the first call per combination of argument shapes; the choice
is kept after that.  Without a GPU tensor among the arguments there is nothing to measure and the batch runs whole.
"""

from __future__ import annotations

import logging

import numpy as np
import torch

from ..vmap import batched_vmap

PROBE_WALKERS = (8, 16)   # allocator granularity (512 B blocks, 2 MB segments) makes probes of 1 and 2 walkers noise


def auto_batched_vmap(fn, in_axes=0, out_axes=0, max_fraction: float = 0.8, max_batch_size: int | None = None):
    """``fn``: a function made by ``forward_laplacian`` / an operator.  ``max_fraction`` of the device memory that is
    free at the first call may be used by one chunk (the reference's default of 1.0 leaves nothing for the results
    of the other chunks, which ``batched_vmap`` keeps until it concatenates them); ``max_batch_size`` caps the choice.
    The chosen chunk sizes are in ``.chosen`` (by argument shapes) of the returned function."""
    chosen: dict = {}

    def walkers_and_device(args):
        axes = tuple(in_axes) if isinstance(in_axes, (tuple, list)) else (in_axes,) * len(args)
        B, dev = None, None
        for a, ax in zip(args, axes):
            if ax is not None and isinstance(a, (torch.Tensor, np.ndarray)):
                B = a.shape[ax] if B is None else B
            if isinstance(a, torch.Tensor) and a.is_cuda:
                dev = a.device
        return B, dev

    def peak_of(n, args, kwargs, dev):
        axes = tuple(in_axes) if isinstance(in_axes, (tuple, list)) else (in_axes,) * len(args)
        part = [a if ax is None or not isinstance(a, (torch.Tensor, np.ndarray))
                else (a.narrow(ax, 0, n) if isinstance(a, torch.Tensor) else np.take(a, range(n), axis=ax))
                for a, ax in zip(args, axes)]
        torch.cuda.synchronize(dev)
        before = torch.cuda.memory_allocated(dev)
        torch.cuda.reset_peak_memory_stats(dev)
        out = batched_vmap(fn, n, in_axes, out_axes)(*part, **kwargs)
        torch.cuda.synchronize(dev)
        peak = torch.cuda.max_memory_allocated(dev) - before
        del out
        return peak

    def result(*args, **kwargs):
        B, dev = walkers_and_device(args)
        key = tuple(tuple(a.shape) if isinstance(a, (torch.Tensor, np.ndarray)) else None for a in args)
        size = chosen.get(key)
        if size is None:
            size = B
            n1, n2 = PROBE_WALKERS
            if dev is not None and B is not None and B > n2:
                try:
                    peak_of(n1, args, kwargs, dev)          # first run: uploads constants, fills the caches
                    p1, p2 = peak_of(n1, args, kwargs, dev), peak_of(n2, args, kwargs, dev)
                    per_walker = max((p2 - p1) / (n2 - n1), 1.0)
                    base = max(p1 - n1 * per_walker, 0.0)
                    free, _ = torch.cuda.mem_get_info(dev)
                    free += torch.cuda.memory_reserved(dev) - torch.cuda.memory_allocated(dev)   # cached, reusable
                    size = int(max((free * max_fraction - base) // per_walker, 1))
                except Exception as e:   # folx/experimental/vmap.py:68-71: fall back to the safest choice
                    logging.warning(f'auto_batched_vmap: could not measure {getattr(fn, "__name__", fn)}: {e}; '
                                    'using chunks of 1')
                    size = 1
            if max_batch_size is not None:
                size = min(size, max_batch_size)
            size = max(min(size, B if B is not None else size), 1)
            chosen[key] = size
        return batched_vmap(fn, size, in_axes, out_axes)(*args, **kwargs)

    result.chosen = chosen
    return result

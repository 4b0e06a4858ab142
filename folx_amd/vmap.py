"""Batching over walkers (``jax.vmap`` in the reference) and chunked batching
(``batched_vmap``, folx/vmap.py:11-83)."""

from __future__ import annotations

import torch


def vmap(fn):
    """``jax.vmap(fn)`` for a function returned by ``forward_laplacian`` or an operator:
    the walker axis is native to the data layout, so this only selects the batched entry."""
    if not hasattr(fn, 'batched'):
        raise TypeError('folx_amd.vmap wraps functions made by forward_laplacian / ForwardLaplacianOperator')
    return fn.batched


def _cat(parts):
    first = parts[0]
    if isinstance(first, tuple):
        return tuple(_cat([p[i] for p in parts]) for i in range(len(first)))
    if isinstance(first, torch.Tensor):
        return torch.cat(parts, dim=0)
    from .api import BatchedArray, FwdJacobian, FwdLaplArray

    if isinstance(first, BatchedArray):
        return BatchedArray(torch.cat([p.data for p in parts], dim=0))
    if isinstance(first, FwdLaplArray):
        return FwdLaplArray(
            torch.cat([p.x for p in parts], 0),
            FwdJacobian(torch.cat([p.jacobian.data for p in parts], 1), first.jacobian.x0_idx),
            torch.cat([p.laplacian for p in parts], 0),
        )
    raise TypeError(type(first))


def batched_vmap(fn, max_batch_size: int):
    """Run ``fn`` over chunks of at most ``max_batch_size`` walkers and concatenate, to
    bound the size of the Jacobian tensors (folx/vmap.py:45-74: full chunks are taken from
    the END of the batch, the remainder -- the first ``B % max`` walkers -- runs on its
    own and is placed first)."""
    batched = vmap(fn)

    def result(x, *args, **kwargs):
        import numpy as np

        B = x.shape[0]
        if B <= max_batch_size:
            return batched(x, *args, **kwargs)
        # every further array argument with the same leading walker axis is chunked along with x
        # (in_axes = 0 of the reference); anything else is passed to every chunk as it is
        walker = [isinstance(a, (torch.Tensor, np.ndarray)) and a.ndim >= 1 and a.shape[0] == B for a in args]
        cut = lambda lo, hi: [a[lo:hi] if w else a for a, w in zip(args, walker)]
        rem = B % max_batch_size
        parts = []
        if rem > 0:
            parts.append(batched(x[:rem], *cut(0, rem), **kwargs))
        for s in range(rem, B, max_batch_size):
            parts.append(batched(x[s : s + max_batch_size], *cut(s, s + max_batch_size), **kwargs))
        return _cat(parts)

    return result

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


def batched_vmap(fn, max_batch_size: int, in_axes=0, out_axes=0):
    """Run ``fn`` over chunks of at most ``max_batch_size`` walkers and concatenate, to
    bound the size of the Jacobian tensors (folx/vmap.py:11-83: full chunks are taken from
    the END of the batch, the remainder -- the first ``B % max`` walkers -- runs on its
    own and is placed first).

    ``in_axes`` as in the reference (and ``jax.vmap``): one entry for all positional arguments
    or one per argument; an int names the walker axis of that argument (moved to the front),
    ``None`` an argument without a walker axis, which is shown whole to every walker.  Nothing
    is inferred from shapes: an array that merely has ``B`` leading entries is only cut when its
    entry of ``in_axes`` says so.  ``out_axes`` must be 0: results keep the walker axis where the
    data layout has it.  The returned function can itself be chunked again over another axis (nested use)
    when it returns tensors."""
    import numpy as np

    if out_axes != 0 and not (isinstance(out_axes, (tuple, list)) and all(a == 0 for a in out_axes)):
        raise NotImplementedError('batched_vmap: out_axes other than 0')
    batched = vmap(fn)

    def result(*args, **kwargs):
        axes = tuple(in_axes) if isinstance(in_axes, (tuple, list)) else (in_axes,) * len(args)
        assert len(axes) == len(args), f'batched_vmap: {len(axes)} in_axes for {len(args)} arguments'
        is_arr = lambda a: isinstance(a, (torch.Tensor, np.ndarray))
        lead = []
        for a, ax in zip(args, axes):
            if ax is None or not is_arr(a):
                lead.append(a)
            else:
                lead.append(a if ax == 0 else (a.movedim(ax, 0) if isinstance(a, torch.Tensor) else np.moveaxis(a, ax, 0)))
        mapped = [a for a, ax in zip(lead, axes) if ax is not None and is_arr(a)]
        assert mapped, 'batched_vmap: no argument carries a walker axis'
        B = mapped[0].shape[0]
        assert all(a.shape[0] == B for a in mapped), 'batched_vmap: walker axes differ in length'

        def cut(lo, hi):
            out = []
            for a, ax in zip(lead, axes):
                if not is_arr(a):
                    out.append(a)
                elif ax is None:   # the same array for every walker of the chunk
                    out.append(a[None].expand(hi - lo, *a.shape) if isinstance(a, torch.Tensor)
                               else np.broadcast_to(a[None], (hi - lo, *a.shape)))
                else:
                    out.append(a[lo:hi])
            return out

        if B <= max_batch_size:
            return batched(*cut(0, B), **kwargs)
        rem = B % max_batch_size
        parts = []
        if rem > 0:
            parts.append(batched(*cut(0, rem), **kwargs))
        for s in range(rem, B, max_batch_size):
            parts.append(batched(*cut(s, s + max_batch_size), **kwargs))
        return _cat(parts)

    def nested(*args, **kwargs):
        """This chunked function under an OUTER ``vmap`` / ``batched_vmap`` (test/test_vmap.py:50-66): every
        array argument arrives with the outer axis in front.  The two axes are flattened into one walker
        axis (an argument that the inner level shows whole is repeated for the inner walkers), the
        flattened batch runs in chunks, and the results get both axes back."""
        axes = tuple(in_axes) if isinstance(in_axes, (tuple, list)) else (in_axes,) * len(args)
        assert len(axes) == len(args), f'batched_vmap: {len(axes)} in_axes for {len(args)} arguments'
        is_arr = lambda a: isinstance(a, (torch.Tensor, np.ndarray))
        outer = [a.shape[0] for a in args if is_arr(a)]
        inner = [a.shape[ax + 1] for a, ax in zip(args, axes) if is_arr(a) and ax is not None]
        assert outer and inner, 'batched_vmap: no argument carries a walker axis'
        Bo, Bi = outer[0], inner[0]
        assert all(b == Bo for b in outer) and all(b == Bi for b in inner), 'batched_vmap: walker axes differ in length'
        flat = []
        for a, ax in zip(args, axes):
            if not is_arr(a):
                flat.append(a)
                continue
            t = a if isinstance(a, torch.Tensor) else torch.as_tensor(np.ascontiguousarray(a))
            t = t[:, None].expand(Bo, Bi, *t.shape[1:]) if ax is None else t.movedim(ax + 1, 1)
            t = t.reshape(Bo * Bi, *t.shape[2:])
            flat.append(t if isinstance(a, torch.Tensor) else t.numpy())
        out = batched_vmap(fn, max_batch_size)(*flat, **kwargs)

        def unflatten(o):
            if isinstance(o, (tuple, list)):
                return type(o)(unflatten(v) for v in o)
            if isinstance(o, torch.Tensor):
                return o.reshape(Bo, Bi, *o.shape[1:])
            raise NotImplementedError('nested batched_vmap: results must be tensors (apply an operator, or take .x / '
                                      '.laplacian / .jacobian.dense_array inside the function)')
        return unflatten(out)

    result.batched = nested
    return result

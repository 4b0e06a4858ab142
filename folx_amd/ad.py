"""Full derivatives of a torch function with the shapes of folx/ad.py:64-107: ``jacrev`` flattens the OUTPUT
(result ``(out.size, *x.shape)`` per argument), ``jacfwd`` flattens the INPUTS (result ``(*out.shape, n_in)`` with
``n_in`` the total size of all arguments), ``hessian = jacfwd(jacrev(f))``.  Real dtypes only.  They are for checks and
small functions -- the forward Laplacian never forms these arrays."""

from __future__ import annotations

import torch
from torch.func import jvp, vjp, vmap

__all__ = ['jacrev', 'jacfwd', 'hessian']


def _tensors(primals):
    return tuple(p if isinstance(p, torch.Tensor) else torch.as_tensor(p) for p in primals)


def jacrev(f):
    """folx/ad.py:64-84: one reverse pass per output entry."""
    def jacfun(*primals):
        primals = _tensors(primals)
        out, pull = vjp(lambda *z: f(*z).reshape(-1), *primals)
        eye = torch.eye(out.numel(), dtype=out.dtype, device=out.device)
        rows = vmap(pull)(eye)                     # one (out.size, *x.shape) per argument
        return rows[0] if len(primals) == 1 else rows

    return jacfun


def jacfwd(f):
    """folx/ad.py:87-102: one forward pass per input entry, the inputs flattened and concatenated on the LAST axis."""
    def jacfun(*primals):
        primals = _tensors(primals)
        sizes = [p.numel() for p in primals]
        n = sum(sizes)
        eye = torch.eye(n, dtype=primals[0].dtype, device=primals[0].device)

        def push(s):
            parts = torch.split(s, sizes)
            return jvp(f, primals, tuple(t.reshape(p.shape) for t, p in zip(parts, primals)))[1]

        return vmap(push, out_dims=-1)(eye)

    return jacfun


def hessian(f):
    """folx/ad.py:105-107."""
    return jacfwd(jacrev(f))

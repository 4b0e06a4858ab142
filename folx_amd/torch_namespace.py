"""The operator namespace of ``folx_amd.workloads`` written with PLAIN TORCH: ``forward(params, r, xp=torch_namespace)``
is then ordinary torch code (differentiable, one sample in), which ``folx_amd.forward_laplacian_torch`` traces and
evaluates through the rules -- the benchmark models through the traced front door, for ``bench.py --front-door torch``
and the tests that compare the two front doors."""

from __future__ import annotations

import numpy as np
import torch

from .fx import multi_head_self_attention  # one traced equation -> the attention rule


def _t(v, like=None):
    if isinstance(v, torch.Tensor):
        return v
    ref = like if isinstance(like, torch.Tensor) else None
    return torch.as_tensor(np.asarray(v), dtype=ref.dtype if ref is not None else torch.float32,
                           device=ref.device if ref is not None else None)


def _pair(a, b):
    return (a if isinstance(a, torch.Tensor) else _t(a, b)), (b if isinstance(b, torch.Tensor) else _t(b, a))


add = lambda a, b: torch.add(*_pair(a, b))
subtract = lambda a, b: torch.sub(*_pair(a, b))
multiply = lambda a, b: torch.mul(*_pair(a, b))
divide = lambda a, b: torch.div(*_pair(a, b))
tanh, silu, sqrt, rsqrt, square, exp, log, sin, cos = (torch.tanh, torch.nn.functional.silu, torch.sqrt, torch.rsqrt,
                                                       torch.square, torch.exp, torch.log, torch.sin, torch.cos)


def dot(h, W, b=None):
    y = h @ _t(W, h)
    return y if b is None else y + _t(b, h)


def layer_norm(h, gamma=None, beta=None, eps=1e-5):
    return torch.nn.functional.layer_norm(h, (h.shape[-1],), None if gamma is None else _t(gamma, h),
                                          None if beta is None else _t(beta, h), eps)


def sum(a, axis=None, keepdims=False):  # noqa: A001 (the namespace mirrors numpy's names)
    return a.sum() if axis is None else a.sum(dim=axis, keepdim=keepdims)


def mean(a, axis=None, keepdims=False):
    return a.mean() if axis is None else a.mean(dim=axis, keepdim=keepdims)


reshape = lambda a, shape: a.reshape(tuple(shape))
transpose = lambda a, axes: a.permute(*axes)
expand_dims = lambda a, axis: a.unsqueeze(axis)
broadcast_to = lambda a, shape: a.expand(*shape)
getitem = lambda a, idx: a[idx]


def concatenate(arrs, axis=-1):
    like = [t for t in arrs if isinstance(t, torch.Tensor)][0]
    return torch.cat([_t(t, like) for t in arrs], dim=axis)


def exp_envelope(d, sigma, pi):
    """``sum_I pi[I, o] exp(-sigma[I, o] d[..., I])`` (broadcast, scale, exp, scale, sum)."""
    return (torch.exp(-d.unsqueeze(-1) * _t(sigma, d)) * _t(pi, d)).sum(dim=-2)


def slogdet(A):
    return torch.linalg.slogdet(A)


def logsumexp(a, axis=-1, b=None):
    """``jax.nn.logsumexp(a, axis, b=b, return_sign=True)``: the shift by the maximum carries no derivative."""
    m = a.amax(dim=axis, keepdim=True).detach()
    e = torch.exp(a - m)
    if b is not None:
        e = e * b
    s = e.sum(dim=axis)
    return torch.log(torch.abs(s)) + m.reshape(s.shape), torch.sign(s)

"""Laplacian operators (folx/operators.py:27-79)."""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Callable, Protocol

from .interpreter import forward_laplacian


class Laplacian(Protocol):
    """folx/operators.py:19-20: ``x -> (laplacian, jacobian)``."""

    def __call__(self, x: Any) -> tuple: ...


class LaplacianOperator(Protocol):
    """folx/operators.py:23-24: ``f -> Laplacian``."""

    def __call__(self, f: Callable) -> Laplacian: ...


class _Laplacian:
    """``lap(x) -> (laplacian, jacobian.dense_array)`` for one sample; ``.batched`` for
    ``(B, *shape)`` walkers (returns laplacian ``(B, ...)`` and Jacobian ``(B, n_in, ...)``
    -- the layout ``jax.vmap`` gives the reference's operator)."""

    def __init__(self, fwd):
        self.fwd = fwd

    def batched(self, x):
        result = self.fwd.batched(x)
        jac = result.jacobian.dense_array  # (n_in, B, ...)
        return result.laplacian, jac.transpose(0, 1)

    def __call__(self, x):
        result = self.fwd(x)
        return result.laplacian[0], result.jacobian.dense_array[:, 0]


@dataclass(frozen=True)
class ForwardLaplacianOperator:
    """folx/operators.py:27-38."""

    sparsity_threshold: float | int

    def __call__(self, f):
        return _Laplacian(forward_laplacian(f, self.sparsity_threshold))


class _DirectionalLaplacian:
    """``lap(x) -> (d2f/dx_i^2 for every input coordinate i, df/dx)`` of a scalar function,
    the return value of the reference's Loop and Parallel operators (folx/operators.py:41-79:
    the diagonal of the Hessian, not its trace, and the gradient).

    Each coordinate is one forward pass with a single Jacobian row ``e_i`` and a zero
    Laplacian: the triplet that arrives at the output is ``(f, df/dx_i, d2f/dx_i^2)``.  The
    passes run through the same rules and kernels as the forward Laplacian, but the sum
    over coordinates happens outside of them, which makes this an independent check of
    every reduction over Jacobian rows.  ``parallel`` stacks the n passes along the walker
    axis and runs them as one."""

    def __init__(self, f, parallel: bool):
        self.fwd = forward_laplacian(f, 0)
        self.parallel = parallel

    def batched(self, x):
        import numpy as np
        import torch

        from . import sparse_ops as so
        from .api import FwdJacobian, FwdLaplArray
        from .interpreter import _device

        dev = _device()
        x = torch.as_tensor(x, dtype=torch.float32).to(dev).contiguous()
        B = x.shape[0]
        shape = tuple(x.shape[1:])
        n = int(np.prod(shape, dtype=int))
        if self.parallel:
            xr = x.repeat_interleave(n, dim=0)  # walker b, direction i -> row b * n + i
            eye = so.device_const(np.eye(n, dtype=np.float32).reshape(1, n, *shape), dev)
            J = eye.expand(B, n, *shape).reshape(1, B * n, *shape).contiguous()
            out = self.fwd.batched(FwdLaplArray(xr, FwdJacobian(J, None), so.zeros(xr.shape, dev)))
            self._check_scalar(out)
            return out.laplacian.reshape(B, n), out.jacobian.dense_array.reshape(B, n)
        laps, jacs = [], []
        for i in range(n):
            e = np.zeros((1, 1, n), dtype=np.float32)
            e[0, 0, i] = 1.0
            J = so.device_const(e.reshape(1, 1, *shape), dev).expand(1, B, *shape).contiguous()
            out = self.fwd.batched(FwdLaplArray(x, FwdJacobian(J, None), so.zeros(x.shape, dev)))
            self._check_scalar(out)
            laps.append(out.laplacian.reshape(B))
            jacs.append(out.jacobian.dense_array.reshape(B))
        return torch.stack(laps, 1), torch.stack(jacs, 1)

    @staticmethod
    def _check_scalar(out):
        if out.shape != ():
            raise ValueError('Loop / Parallel Laplacian operators take scalar functions (the reference uses jax.grad)')

    def __call__(self, x):
        lap, jac = self.batched(x[None])
        return lap[0], jac[0]


class LoopLaplacianOperator:
    """folx/operators.py:41-62: one pass per input coordinate."""

    @staticmethod
    def __call__(f):
        return _DirectionalLaplacian(f, parallel=False)


class ParallelLaplacianOperator:
    """folx/operators.py:65-79: all coordinates in one pass."""

    @staticmethod
    def __call__(f):
        return _DirectionalLaplacian(f, parallel=True)

"""Laplacian operators (folx/operators.py:27-79)."""

from __future__ import annotations

from dataclasses import dataclass

from .interpreter import forward_laplacian


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

"""Front door: ``forward_laplacian(fn, sparsity_threshold)``.

The reference traces ``fn`` to a jaxpr and interprets it once under ``jax.jit``
(folx/interpreter.py:301-352).  Here ``fn`` is written against ``folx_amd.numpy`` and runs
define-by-run on ``FwdLaplArray`` triplets; batching over walkers, which the reference
gets from an outer ``jax.vmap``, is built into the data layout and switched on with
``folx_amd.vmap`` / ``batched_vmap``.
"""

from __future__ import annotations

import numpy as np
import torch

from . import index_algebra as ia
from . import numpy as fnp
from . import sparse_ops as so
from .api import BatchedArray, FwdJacobian, FwdLaplArray


def _device():
    if not torch.cuda.is_available():
        from ._lib import FolxHipError

        raise FolxHipError('folx_amd needs a GPU: the forward Laplacian runs in HIP kernels only')
    return torch.device('cuda', torch.cuda.current_device())


def init_forward_laplacian_state(x: torch.Tensor, sparsity: bool, weights=None, offset: int = 0,
                                 total: int | None = None) -> FwdLaplArray:
    """Initial triplet for an input ``x (B, *shape)`` (folx/interpreter.py:267-298):
    sparse -> one row holding the weights with ``x0_idx = arange(n).reshape(shape)``
    (:286-293); dense -> ``diag(weights)`` reshaped to ``(n, *shape)`` (:295); lap = 0.

    With several differentiated arguments the inputs share one index space, numbered in
    argument order (the reference flattens the argument tree, :331-340): this argument's
    coordinates are ``offset .. offset + n`` of ``total``."""
    B = x.shape[0]
    shape = tuple(x.shape[1:])
    n = int(np.prod(shape, dtype=int))
    total = n if total is None else int(total)
    dev = x.device
    w = np.ones(shape, dtype=np.float32) if weights is None else np.broadcast_to(
        np.asarray(weights, dtype=np.float32), shape)
    lap = so.zeros(x.shape, dev)
    if sparsity:
        data = so.device_const(np.ascontiguousarray(w), dev).reshape(1, 1, *shape).expand(1, B, *shape).contiguous()
        return FwdLaplArray(x, FwdJacobian(data, ia.init_mask(shape, offset)), lap)
    eye = np.zeros((total, n), dtype=np.float32)
    eye[offset:offset + n] = np.eye(n, dtype=np.float32) * w.reshape(-1)
    data = so.device_const(eye.reshape(total, 1, *shape), dev).expand(total, B, *shape).contiguous()
    return FwdLaplArray(x, FwdJacobian(data, None), lap)


def _force_tree(out):
    """Evaluate whatever the function returned unevaluated (``wrapped_functions.Deferred``)."""
    from .wrapped_functions import Deferred

    if isinstance(out, Deferred):
        return out.value()
    if isinstance(out, (tuple, list)):
        return type(out)(_force_tree(t) for t in out)
    if isinstance(out, dict):
        return {k: _force_tree(v) for k, v in out.items()}
    return out


class ForwardLaplacianFn:
    """Callable returned by ``forward_laplacian``.  ``f(x)`` treats ``x`` as ONE sample of
    shape ``shape`` (the reference's un-vmapped call); ``f.batched(x)`` takes
    ``(B, *shape)`` walkers -- what ``jax.vmap(f)`` is in the reference."""

    def __init__(self, fn, sparsity_threshold):
        self.fn = fn
        self.sparsity_threshold = sparsity_threshold

    def _threshold(self, size: int) -> int:
        t = self.sparsity_threshold
        if 0 < t < 1:  # fraction of the input size (folx/interpreter.py:333-336)
            return int(t * size)
        return int(t)

    def batched(self, *args, weights=None, **kwargs):
        dev = _device()
        lapl_args = []
        size = 0
        for a in args:
            if isinstance(a, (FwdLaplArray, BatchedArray)):
                size += int(np.prod(a.shape, dtype=int))
            elif isinstance(a, (torch.Tensor, np.ndarray)):
                size += int(np.prod(a.shape[1:], dtype=int))
        thr = self._threshold(size)
        # several array arguments are differentiated together: one index space, numbered in argument order
        sizes = [int(np.prod(a.shape[1:], dtype=int)) if isinstance(a, (torch.Tensor, np.ndarray)) else 0 for a in args]
        total, offset = int(np.sum(sizes)), 0
        if isinstance(weights, (tuple, list)):
            assert len(weights) == len(args), 'weights: one entry per argument'
        for i, a in enumerate(args):
            if isinstance(a, (FwdLaplArray, BatchedArray)):
                lapl_args.append(a)
            elif isinstance(a, (torch.Tensor, np.ndarray)):
                x = torch.as_tensor(a, dtype=torch.float32).to(dev).contiguous()
                w = weights[i] if isinstance(weights, (tuple, list)) else weights
                lapl_args.append(init_forward_laplacian_state(x, thr > 0, w, offset, total))
                offset += sizes[i]
            else:
                lapl_args.append(a)
        with fnp.sparsity_threshold(thr):
            return _force_tree(self.fn(*lapl_args, **kwargs))

    def __call__(self, *args, weights=None, **kwargs):
        lifted = []
        for a in args:
            if isinstance(a, torch.Tensor):
                lifted.append(a[None])
            elif isinstance(a, np.ndarray) or np.isscalar(a):
                lifted.append(np.asarray(a)[None])
            else:
                lifted.append(a)
        return self.batched(*lifted, weights=weights, **kwargs)


def forward_laplacian(fn, sparsity_threshold: int | float = 0, disable_jit: bool = False) -> ForwardLaplacianFn:
    """folx/interpreter.py:301-352.  ``sparsity_threshold`` in (0, 1) is a fraction of the
    input size; 0 disables sparse Jacobians.  ``disable_jit`` is accepted for signature
    parity (execution is always eager; a HIP graph can be captured around the call)."""
    del disable_jit
    return ForwardLaplacianFn(fn, sparsity_threshold)

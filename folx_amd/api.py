"""Data model of the forward Laplacian on MI355X: the ``(x, jacobian, laplacian)`` triplet.

Mirrors folx/api.py (``FwdJacobian`` :19-42, ``FwdLaplArray`` :266-274, ``FunctionFlags``
:453-464) with device tensors in the layout the HIP kernels stream:

    x         (B, *shape)        B = walkers (what ``jax.vmap`` adds in the reference)
    jacobian  (P, B, *shape)     Jacobian axis leading (``JAC_DIM = 0``), walkers next
    laplacian (B, *shape)

``shape`` / ``ndim`` of these classes are the per-walker (logical) ones, exactly what a
function sees inside ``jax.vmap``.  The sparsity mask ``x0_idx`` is a host numpy array of
shape ``(k, *shape)`` shared by all walkers, as in the reference under ``vmap``.
"""

from __future__ import annotations

from enum import IntFlag
from typing import Any, NamedTuple, Protocol

import numpy as np
import torch

JAC_DIM = 0  # folx/api.py:16


class FunctionFlags(IntFlag):
    """folx/api.py:453-464."""

    GENERAL = 0
    LINEAR_IN_FIRST = 1 << 0
    LINEAR_IN_ONE = 1 << 1 | LINEAR_IN_FIRST
    LINEAR = 1 << 2 | LINEAR_IN_ONE
    REDUCTION = 1 << 3
    MULTIPLICATION = 1 << 4 | LINEAR_IN_ONE
    DOT_PRODUCT = 1 << 5 | REDUCTION | MULTIPLICATION
    INDEXING = 1 << 6 | LINEAR
    SCATTER = 1 << 7
    SPARSE_JHJ = 1 << 8
    SUMMATION = 1 << 9 | LINEAR | REDUCTION


class BatchedArray:
    """A derivative-free array that differs per walker: ``data (B, *shape)`` on the GPU.
    The reference has no such class -- under ``jax.vmap`` it is an ordinary traced array
    (e.g. the ``sign`` output of slogdet, folx/slogdet.py:344)."""

    __slots__ = ('data',)

    def __init__(self, data: torch.Tensor):
        self.data = data

    @property
    def shape(self):
        return tuple(self.data.shape[1:])

    @property
    def ndim(self):
        return self.data.dim() - 1

    @property
    def B(self):
        return self.data.shape[0]

    def __repr__(self):
        return f'BatchedArray(shape={self.shape}, B={self.B})'


class FwdJacobian:
    """Jacobian w.r.t. the function's initial arguments, dense (``x0_idx is None``, row p
    = input p) or sparse (``k`` rows + host mask naming the input of each entry, ``-1`` =
    none).  folx/api.py:19-42.

    data   : torch.Tensor (k, B, *shape)
    x0_idx : np.ndarray (k, *shape) or None
    """

    __slots__ = ('data', 'x0_idx')

    def __init__(self, data: torch.Tensor, x0_idx: np.ndarray | None = None):
        self.data = data
        self.x0_idx = x0_idx

    def __iter__(self):
        return iter((self.data, self.x0_idx))

    def _replace(self, **kw):
        return FwdJacobian(kw.get('data', self.data), kw.get('x0_idx', self.x0_idx))

    def __repr__(self):
        kind = 'dense' if self.x0_idx is None else 'sparse'
        return f'FwdJacobian({kind}, data={tuple(self.data.shape)})'

    @property
    def weak(self) -> bool:
        return self.x0_idx is not None

    @property
    def unique_idx(self):
        if self.x0_idx is not None:
            return np.unique(self.x0_idx)
        return np.arange(self.data.shape[JAC_DIM])

    @property
    def data_shape(self):
        """Per-walker shape of the array this Jacobian belongs to."""
        return tuple(self.data.shape[2:])

    @property
    def max_n(self) -> int:
        if self.x0_idx is not None:
            return int(np.max(self.x0_idx))
        return self.data.shape[JAC_DIM]

    @property
    def mask(self) -> np.ndarray:
        """folx/api.py:211-220."""
        if self.x0_idx is not None:
            return self.x0_idx
        P = self.data.shape[JAC_DIM]
        shape = self.data_shape
        m = np.arange(P, dtype=np.int32).reshape(P, *([1] * len(shape)))
        return np.broadcast_to(m, (P, *shape))

    def get_index_mask(self, outputs: np.ndarray) -> np.ndarray:
        """folx/api.py:120-159 (host, numpy)."""
        from . import index_algebra as ia

        assert self.weak
        return ia.get_index_mask(self.x0_idx, outputs)

    def materialize_for_idx(self, idx: np.ndarray, max_idx: int) -> torch.Tensor:
        """Sum the rows into ``max_idx`` target rows by the static slot map ``idx``
        (k, *shape); folx/api.py:58-118.  Runs the gather kernel."""
        from . import sparse_ops

        assert self.weak
        return sparse_ops.materialize(self.data, idx, max_idx)

    def construct_jac_for(self, idx):
        """folx/api.py:165-180."""
        if idx is None:
            return self.dense_array
        if len(idx) == 0:
            return self.data.new_zeros((1, *self.data.shape[1:]))
        if self.x0_idx is None:
            return self.data[np.asarray(idx).reshape(-1)].contiguous()
        return self.materialize_for_idx(self.get_index_mask(idx), len(idx))

    @property
    def dense_array(self) -> torch.Tensor:
        """Dense ``(max_n + 1, B, *shape)`` Jacobian (folx/api.py:182-190)."""
        if self.x0_idx is None:
            return self.data
        n_out = self.max_n + 1
        return self.materialize_for_idx(np.maximum(self.x0_idx, -1), n_out)

    @property
    def as_dense(self) -> 'FwdJacobian':
        return FwdJacobian(self.dense_array, None)

    @classmethod
    def from_dense(cls, array):
        return cls(array, None)

    def __add__(self, other):  # type: ignore[override]
        """folx/api.py:230-249."""
        from . import sparse_ops

        assert isinstance(other, FwdJacobian)
        return sparse_ops.add_jacobians(self, other)


class FwdLaplArray:
    """Triplet of a tensor, its Jacobian and its Laplacian (folx/api.py:266-333).

    x         : torch.Tensor (B, *shape)
    jacobian  : FwdJacobian
    laplacian : torch.Tensor (B, *shape)
    """

    __slots__ = ('x', 'jacobian', 'laplacian')

    def __init__(self, x: torch.Tensor, jacobian: FwdJacobian, laplacian: torch.Tensor):
        self.x = x
        self.jacobian = jacobian
        self.laplacian = laplacian

    def __iter__(self):
        return iter((self.x, self.jacobian, self.laplacian))

    def _replace(self, **kw):
        return FwdLaplArray(
            kw.get('x', self.x), kw.get('jacobian', self.jacobian), kw.get('laplacian', self.laplacian)
        )

    def __repr__(self):
        return f'FwdLaplArray(shape={self.shape}, B={self.B}, jacobian={self.jacobian!r})'

    @property
    def shape(self):
        return tuple(self.x.shape[1:])

    @property
    def ndim(self):
        return self.x.dim() - 1

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=int))

    @property
    def B(self):
        return self.x.shape[0]

    @property
    def dtype(self):
        return self.x.dtype

    @property
    def dense_jacobian(self):
        return self.jacobian.dense_array

    @property
    def is_jacobian_weak(self):
        return self.jacobian.weak

    @property
    def sparse_jacobian(self):
        assert self.jacobian.weak
        return self.jacobian.data

    @property
    def jacobian_mask(self):
        return self.jacobian.mask

    @property
    def dense(self):
        return FwdLaplArray(self.x, self.jacobian.as_dense, self.laplacian)

    # ---- operator sugar (the reference gets this from tracing jnp code) ----------------
    # numpy leaves `array <op> triplet` to the reflected methods below instead of broadcasting over the tuple
    __array_ufunc__ = None

    def __add__(self, o):
        from . import numpy as fnp

        return fnp.add(self, o)

    def __radd__(self, o):
        from . import numpy as fnp

        return fnp.add(o, self)

    def __sub__(self, o):
        from . import numpy as fnp

        return fnp.subtract(self, o)

    def __rsub__(self, o):
        from . import numpy as fnp

        return fnp.subtract(o, self)

    def __mul__(self, o):
        from . import numpy as fnp

        return fnp.multiply(self, o)

    def __rmul__(self, o):
        from . import numpy as fnp

        return fnp.multiply(o, self)

    def __truediv__(self, o):
        from . import numpy as fnp

        return fnp.divide(self, o)

    def __rtruediv__(self, o):
        from . import numpy as fnp

        return fnp.divide(o, self)

    def __neg__(self):
        from . import numpy as fnp

        return fnp.negative(self)

    def __matmul__(self, W):
        from . import numpy as fnp

        return fnp.dot(self, W)

    def __getitem__(self, idx):
        from . import numpy as fnp

        return fnp.getitem(self, idx)

    def __rmatmul__(self, W):
        from . import numpy as fnp

        return fnp.matmul(W, self)

    def __pow__(self, e):
        from . import numpy as fnp

        if isinstance(e, (int, np.integer)) and not isinstance(e, bool):
            return fnp.integer_pow(self, int(e))
        return fnp.power(self, e)

    def __rpow__(self, base):
        from . import numpy as fnp

        return fnp.power(base, self)

    def __abs__(self):
        from . import numpy as fnp

        return fnp.abs(self)

    # comparisons give values without derivatives (== and != stay the tuple's own)
    def __gt__(self, o):
        from . import numpy as fnp

        return fnp.greater(self, o)

    def __ge__(self, o):
        from . import numpy as fnp

        return fnp.greater_equal(self, o)

    def __lt__(self, o):
        from . import numpy as fnp

        return fnp.less(self, o)

    def __le__(self, o):
        from . import numpy as fnp

        return fnp.less_equal(self, o)

    @property
    def T(self):
        from . import numpy as fnp

        return fnp.transpose(self, tuple(reversed(range(len(self.shape)))))

    def transpose(self, *axes):
        from . import numpy as fnp

        if len(axes) == 1 and isinstance(axes[0], (tuple, list)):
            axes = tuple(axes[0])
        return fnp.transpose(self, axes if axes else tuple(reversed(range(len(self.shape)))))

    def swapaxes(self, a, b):
        from . import numpy as fnp

        return fnp.swapaxes(self, a, b)

    def mean(self, axis=None, keepdims=False):
        from . import numpy as fnp

        return fnp.mean(self, axis=axis, keepdims=keepdims)
    def reshape(self, *shape):
        from . import numpy as fnp

        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        return fnp.reshape(self, shape)

    def sum(self, axis=None, keepdims=False):
        from . import numpy as fnp

        return fnp.sum(self, axis=axis, keepdims=keepdims)


def IS_LPL_ARR(x):
    return isinstance(x, FwdLaplArray)


class FwdLaplArgs(NamedTuple):
    """folx/api.py:348-409."""

    arrays: tuple

    @property
    def x(self):
        return tuple(a.x for a in self.arrays)

    @property
    def jacobian(self):
        return tuple(a.jacobian for a in self.arrays)

    @property
    def laplacian(self):
        return tuple(a.laplacian for a in self.arrays)

    @property
    def jacobian_mask(self):
        return tuple(a.jacobian_mask for a in self.arrays)

    @property
    def all_jacobian_weak(self) -> bool:
        return all(a.is_jacobian_weak for a in self.arrays)

    @property
    def any_jacobian_weak(self) -> bool:
        return any(a.is_jacobian_weak for a in self.arrays)

    @property
    def dense(self):
        return FwdLaplArgs(tuple(a.dense for a in self.arrays))

    def __len__(self) -> int:
        return len(self.arrays)


class ForwardLaplacian(Protocol):
    """Rule type of the registry (folx/api.py:444-450)."""

    def __call__(self, args: tuple, kwargs: dict[str, Any], sparsity_threshold: int) -> Any: ...

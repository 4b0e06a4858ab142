"""Device side of the sparse-Jacobian bookkeeping: host masks in, gather-kernel launches out.

The index tables built by ``index_algebra`` are uploaded once and cached by content, so a
model that is evaluated repeatedly (or replayed from a HIP graph) never re-uploads them.
"""

from __future__ import annotations

import hashlib

import numpy as np
import torch

from . import index_algebra as ia
from . import kernels as K
from .api import FwdJacobian

class _ByteLRU:
    """Least-recently-used cache of device tensors (or tuples holding some) bounded by bytes: a loop
    that keeps handing over fresh numpy constants or masks cannot grow it without limit.  An entry
    that is dropped stays alive for as long as something else refers to it (a captured HIP graph
    keeps the tensors it reads, ``graph._Captured``)."""

    def __init__(self, max_bytes: int):
        from collections import OrderedDict

        self.max_bytes, self.bytes, self.d = int(max_bytes), 0, OrderedDict()

    @staticmethod
    def _size(v) -> int:
        if isinstance(v, torch.Tensor):
            return v.numel() * v.element_size()
        if isinstance(v, (tuple, list)):
            return sum(_ByteLRU._size(t) for t in v)
        return 0

    def get(self, key, default=None):
        hit = self.d.get(key)
        if hit is None:
            return default
        self.d.move_to_end(key)
        return hit

    def __setitem__(self, key, value):
        if key in self.d:
            self.bytes -= self._size(self.d[key])
        self.d[key] = value
        self.d.move_to_end(key)
        self.bytes += self._size(value)
        while self.bytes > self.max_bytes and len(self.d) > 1:
            _, old = self.d.popitem(last=False)
            self.bytes -= self._size(old)

    def __len__(self):
        return len(self.d)

    def values(self):
        return list(self.d.values())

    def clear(self):
        self.d.clear()
        self.bytes = 0


_TABLE_CACHE = _ByteLRU(1 << 30)   # int32 gather / scatter tables, keyed by the content of the host mask
_CONST_CACHE = _ByteLRU(1 << 30)   # float32 constants and numpy weights, keyed by content
_MAX_TABLE_ENTRIES = 1 << 27  # beyond this the scatter-add kernel is used instead


def _key(arr: np.ndarray, *extra):
    a = np.asarray(arr)
    # the shape is the ARGUMENT's: numpy.ascontiguousarray turns a 0-d array into shape (1,), and a scalar constant
    # must not share its entry with a one-element vector of the same value
    return (hashlib.blake2b(np.ascontiguousarray(a).tobytes(), digest_size=16).digest(), a.shape, str(a.dtype), *extra)


def device_table(arr: np.ndarray, device) -> torch.Tensor:
    """int32 table on the device, cached by content."""
    key = _key(arr, 'i32', str(device))
    t = _TABLE_CACHE.get(key)
    if t is None:
        # a copy: the source may be one of the read-only masks, which torch would warn about wrapping
        t = torch.from_numpy(np.array(arr, dtype=np.int32, order='C')).to(device)
        _TABLE_CACHE[key] = t
    return t


def device_const(arr, device) -> torch.Tensor:
    """float32 constant on the device; numpy inputs are cached by content."""
    if isinstance(arr, torch.Tensor):
        if arr.device != device or arr.dtype != torch.float32:
            arr = arr.to(device=device, dtype=torch.float32)
        return arr.contiguous()
    a = np.array(arr, dtype=np.float32, order='C', copy=True)
    key = _key(a, 'f32', str(device))
    t = _CONST_CACHE.get(key)
    if t is None:
        t = torch.as_tensor(a).to(device)
        _CONST_CACHE[key] = t
    return t


def cached_tensors() -> list:
    """Every device tensor the caches hold right now (what a captured graph must keep alive)."""
    out = []
    for v in _TABLE_CACHE.values() + _CONST_CACHE.values() + [r[1] for r in _ROWS_CACHE.values()]:
        out.extend(t for t in (v if isinstance(v, (tuple, list)) else (v,)) if isinstance(t, torch.Tensor))
    return out


def clear_caches():
    from . import index_algebra

    _TABLE_CACHE.clear()
    _CONST_CACHE.clear()
    _ROWS_CACHE.clear()
    index_algebra._MEMO.clear()
    index_algebra._BY_IDENTITY.clear()


def zeros(shape, device) -> torch.Tensor:
    """Zero tensor produced by a fill kernel (never by a memset node, so that the call can
    sit inside a captured HIP graph)."""
    return torch.empty(shape, device=device, dtype=torch.float32).zero_()


def materialize(data: torch.Tensor, idx: np.ndarray, n_out: int) -> torch.Tensor:
    """out[t, b, pos] = sum of data[r, b, pos] over rows r with idx[r, pos] == t.

    data (k, B, *s) on the device, idx (k, *s) host slot map (``-1`` = drop).  Static
    gather (folx/utils.py:71-114) through ``folx_hip_gather_rows``; the table is stored
    without the trailing axes along which ``idx`` is constant.
    """
    k, B = data.shape[0], data.shape[1]
    s = tuple(data.shape[2:])
    idx = np.broadcast_to(idx, (k, *s))
    if n_out == 0 or k == 0:
        return zeros((n_out, B, *s), data.device)
    n_inner = ia.split_inner(idx)
    n_outer_axes = len(s) - n_inner
    s_outer, s_inner = s[:n_outer_axes], s[n_outer_axes:]
    S_outer = int(np.prod(s_outer, dtype=np.int64))
    S_inner = int(np.prod(s_inner, dtype=np.int64))
    idx_c = idx[(slice(None), *([slice(None)] * n_outer_axes), *([0] * n_inner))]
    data = data.contiguous().reshape(k, B, S_outer * S_inner)
    key = _key(idx_c, 'take', n_out)
    cached = _TABLE_CACHE.get((key, str(data.device)))
    if cached is None:
        take = ia.gather_table(idx_c, n_out)
        n_slots = take.shape[1]
        # The gather kernel writes every output entry exactly once, in memory order (5.9 TB/s also for a
        # mostly empty result: k = 3 of 96 rows at 1024 x 32 x 256 in 0.56 ms; a fill followed by an atomic
        # scatter of the rows that exist takes 0.58 ms and depends on the order of colliding additions).
        # Only a table past _MAX_TABLE_ENTRIES -- 512 MiB of int32 -- takes the scatter form: its result is
        # then exact up to the order of the atomic additions, i.e. to rounding.
        if take.size > _MAX_TABLE_ENTRIES:
            cached = ('scatter', device_table(idx_c.reshape(k, S_outer), data.device), 0)
        else:
            cached = ('gather', device_table(take.reshape(n_out, n_slots, S_outer), data.device), n_slots)
        _TABLE_CACHE[(key, str(data.device))] = cached
    kind, table, n_slots = cached
    if kind == 'gather':
        out = K.gather_rows(data, table, n_out, n_slots, B, S_outer, S_inner)
    else:
        out = K.scatter_add_rows(data, table, n_out, B, S_outer, S_inner)
    return out.reshape(n_out, B, *s)


def materialize_reduced(data: torch.Tensor, slot: np.ndarray, n_out: int, axis: int, shape, window=None,
                        alpha: float = 1.0) -> torch.Tensor:
    """``alpha * sum`` over logical axis ``axis`` (its window ``[lo, hi)``) of sparse rows into their
    output slots: out[t, b, kept] = alpha * sum of data[r, b, .., j, ..] over (r, j) with
    slot[r, .., j, ..] == t (folx/jvp.py:144-171).  data (k, B, *shape) is read where it lies
    (``folx_hip_gather_reduce_rows``); ``slot`` (k, *shape) with the window already cut out of the
    reduced axis when ``window`` is given."""
    k, B = data.shape[0], data.shape[1]
    shape = tuple(shape)
    RED = shape[axis]
    lo, hi = (0, RED) if window is None else window
    before, after = shape[:axis], shape[axis + 1:]
    if n_out == 0 or k == 0 or hi == lo:
        return zeros((n_out, B, *before, *after), data.device)
    # (k * RED, *kept) slot map with the row id r * RED + j; entries outside the window name no slot
    full = np.full((k, *before, RED, *after), -1, dtype=np.int32)
    full[(slice(None), *([slice(None)] * axis), slice(lo, hi))] = slot
    sp = np.moveaxis(full, axis + 1, 1).reshape(k * RED, *before, *after)
    n_const = min(ia.split_inner(sp), len(after))  # trailing kept axes along which the map is constant
    n_var = len(after) - n_const
    O = int(np.prod(before, dtype=np.int64))
    IV = int(np.prod(after[:n_var], dtype=np.int64))
    IC = int(np.prod(after[n_var:], dtype=np.int64))
    idx_c = sp[(slice(None), *([slice(None)] * (len(before) + n_var)), *([0] * n_const))]
    key = _key(np.ascontiguousarray(idx_c), 'take_reduced', n_out)
    cached = _TABLE_CACHE.get((key, str(data.device)))
    if cached is None:
        take = ia.gather_table(idx_c, n_out)
        cached = (device_table(take.reshape(n_out, take.shape[1], O * IV), data.device), take.shape[1])
        _TABLE_CACHE[(key, str(data.device))] = cached
    table, n_slots = cached
    out = K.gather_reduce_rows(data.contiguous(), table, n_out, n_slots, B, O, RED, IV, IC, alpha)
    return out.reshape(n_out, B, *before, *after)


def pad_rows(data: torch.Tensor, P: int) -> torch.Tensor:
    """Zero-extend a dense Jacobian to P rows (folx/utils.py:432-450)."""
    if data.shape[0] == P:
        return data
    out = torch.empty((P, *data.shape[1:]), device=data.device, dtype=data.dtype)
    out[: data.shape[0]].copy_(data)
    out[data.shape[0] :].zero_()
    return out


def add_rowstacks(a: torch.Tensor, b: torch.Tensor, sign: float = 1.0) -> torch.Tensor:
    """a + sign * b for two equally shaped row stacks (one flat affine launch)."""
    n = a.numel()
    out = K.rows_affine(a.contiguous(), 1, (n,), (n,), None, b.contiguous().reshape(n), 1.0, sign)
    return out.reshape(a.shape)


def add_jacobians(a: FwdJacobian, b: FwdJacobian) -> FwdJacobian:
    """``FwdJacobian.__add__`` (folx/api.py:230-249)."""
    if not a.weak or not b.weak:
        da, db = a.dense_array, b.dense_array
        P = max(da.shape[0], db.shape[0])
        return FwdJacobian(add_rowstacks(pad_rows(da, P), pad_rows(db, P)), None)
    if a.x0_idx.shape[0] == b.x0_idx.shape[0] and np.array_equal(
        *np.broadcast_arrays(a.x0_idx, b.x0_idx)
    ):
        return FwdJacobian(add_rowstacks(a.data, b.data), np.broadcast_arrays(a.x0_idx, b.x0_idx)[0])
    return FwdJacobian(
        torch.cat([a.data, b.data], dim=0), np.concatenate([a.x0_idx, b.x0_idx], axis=0)
    )


def add_sparse_rows_(dense: torch.Tensor, data: torch.Tensor, idx: np.ndarray) -> None:
    """dense[idx[r, pos], b, pos] += data[r, b, pos], in place: adds a sparse Jacobian
    (``data (k, B, *s)``, mask ``idx (k, *s)``, ``-1`` = no entry) into a dense row stack
    ``(P, B, *s)`` that the caller owns (e.g. the fresh output of a GEMM), touching only the
    k stored rows instead of materialising them first."""
    k, B = data.shape[0], data.shape[1]
    s = tuple(data.shape[2:])
    idx = np.broadcast_to(idx, (k, *s))
    n_inner = ia.split_inner(idx)
    n_outer_axes = len(s) - n_inner
    S_outer = int(np.prod(s[:n_outer_axes], dtype=np.int64))
    S_inner = int(np.prod(s[n_outer_axes:], dtype=np.int64))
    idx_c = idx[(slice(None), *([slice(None)] * n_outer_axes), *([0] * n_inner))]
    assert int(idx_c.max(initial=-1)) < dense.shape[0]
    table = device_table(idx_c.reshape(k, S_outer), data.device)
    P = dense.shape[0]
    K.scatter_add_rows(data.contiguous().reshape(k, B, S_outer * S_inner), table, P, B, S_outer, S_inner,
                       out=dense.reshape(P, B, S_outer * S_inner))


_ROWS_CACHE: dict = {}


def weight_rows(W: torch.Tensor, ranges: tuple, cache: bool = False) -> torch.Tensor:
    """Rows ``[lo, hi)`` of a weight matrix for each range, concatenated (a contiguous copy unless one
    range covers it).  ``cache``: only for a ``W`` that this module made from a numpy constant
    (``device_const``, never written again): the copy is then kept per (tensor object, ranges).  A
    tensor the caller owns may be updated in place at any time -- also between the replays of a
    captured graph, which would go on reading a cached copy -- so its rows are copied on every
    call, and a capture records that copy."""
    import weakref

    if len(ranges) == 1:
        lo, hi = ranges[0]
        return W[lo:hi]  # consecutive rows of a row-major matrix are contiguous
    if not cache:
        return torch.cat([W[lo:hi] for lo, hi in ranges], dim=0)
    key = (id(W), ranges)
    hit = _ROWS_CACHE.get(key)
    if hit is not None and hit[0]() is W:
        return hit[1]
    if len(_ROWS_CACHE) >= 64:
        _ROWS_CACHE.pop(next(iter(_ROWS_CACHE)))
    rows = torch.cat([W[lo:hi] for lo, hi in ranges], dim=0).contiguous()
    _ROWS_CACHE[key] = (weakref.ref(W), rows)
    return rows

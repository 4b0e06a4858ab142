"""Static sparsity algebra on the host (numpy, integers only).

Sparse Jacobians carry a compile-time mask ``x0_idx (k, *shape)``; every rule has to say
what the mask of its output is and how input rows map to output rows.  The functions here
compute those maps, vectorised over positions, and turn them into the small int32 tables
the gather kernel consumes.  They mirror the reference's host-side helpers; each cites the
lines it follows.  Nothing here touches the GPU.
"""

from __future__ import annotations

from typing import Sequence

import numpy as np

INT = np.int64

# The maps below depend on the masks' contents only, and a model asks for the same ones at
# every evaluation: results are kept by content (the reference gets the same effect from
# tracing once under jit).  Cached arrays are shared between callers and read-only.
_MEMO: dict = {}
_MEMO_MAX = 1024


def _freeze(v):
    """Results of the memoized functions are values: read-only, and so is the memory they are views of (masks
    are never written in place anywhere in this package)."""
    if isinstance(v, np.ndarray):
        b = v
        while isinstance(b, np.ndarray):
            b.flags.writeable = False
            b = b.base
    elif isinstance(v, tuple):
        for t in v:
            _freeze(t)
    return v


def _stable(v: np.ndarray) -> bool:
    """Nobody can write to the memory of ``v``: the array and everything it is a view of are read-only."""
    while isinstance(v, np.ndarray):
        if v.flags.writeable:
            return False
        v = v.base
    return v is None


def _key_of(v):
    if isinstance(v, np.ndarray):
        return ('a', v.shape, v.dtype.str, np.ascontiguousarray(v).tobytes())  # exact: the contents are the key
    if isinstance(v, (list, tuple)):
        return tuple(_key_of(t) for t in v)
    if isinstance(v, np.generic):
        return v.item()
    return v


_BY_IDENTITY: dict = {}


def _identity_key(args):
    """Key of an argument list by the MEMORY of its read-only arrays (address, shape, strides, type: two views of
    one cached mask with the same layout are the same value), or None when some array could still be written to
    (its address says nothing about its contents then) or an argument has no cheap key."""
    key = []
    for v in args:
        if isinstance(v, np.ndarray):
            if not _stable(v):
                return None
            key.append(('m', v.__array_interface__['data'][0], v.shape, v.strides, v.dtype.str))
        elif isinstance(v, (list, tuple)):
            sub = _identity_key(v)
            if sub is None:
                return None
            key.append(sub)
        elif v is None or isinstance(v, (bool, int, float, str, np.generic)):
            key.append(v.item() if isinstance(v, np.generic) else v)
        else:
            return None
    return tuple(key)


def _memo(fn):
    """Keeps results of a pure function of integer arrays and plain values by content.  Results are read-only
    arrays that the next rule receives as they are, so from the second evaluation of a model on its masks ARE the
    cached objects or views of them: a first look-up by the memory of read-only arguments (an entry keeps its arguments
    alive, so an address cannot be reused while it is a key) saves building and hashing a key of the contents."""
    import functools

    @functools.wraps(fn)
    def wrapped(*args):
        ikey = _identity_key(args)
        if ikey is not None:
            hit = _BY_IDENTITY.get((fn.__name__, ikey))
            if hit is not None:
                return hit[1]
        key = (fn.__name__, _key_of(args))
        hit = _MEMO.get(key)
        if hit is None:
            if len(_MEMO) >= _MEMO_MAX:
                _MEMO.clear()
                _BY_IDENTITY.clear()
            hit = _MEMO[key] = _freeze(fn(*args))
        if ikey is not None:
            if len(_BY_IDENTITY) >= 4 * _MEMO_MAX:
                _BY_IDENTITY.clear()
            _BY_IDENTITY[(fn.__name__, ikey)] = (args, hit)
        return hit

    return wrapped


# --------------------------------------------------------------------------------------
# small helpers
# --------------------------------------------------------------------------------------


def init_mask(shape, offset: int = 0) -> np.ndarray:
    """Initial sparse mask: one row, entry i <- flat input ``offset + i`` (folx/interpreter.py:283-293).  The same
    read-only array for the same shape, so that everything derived from it is found by identity."""
    return _init_mask(tuple(int(n) for n in shape), int(offset))


@_memo
def _init_mask(shape, offset):
    n = int(np.prod(shape, dtype=int))
    return (np.arange(n, dtype=np.int32) + np.int32(offset)).reshape(1, *shape)


@_memo
def has_duplicates(mask: np.ndarray | None) -> bool:
    """True iff a position lists a valid index twice (folx/hessian.py:71-84)."""
    if mask is None or mask.shape[0] <= 1:
        return False
    s = np.sort(mask, axis=0)
    return bool(((s[1:] == s[:-1]) & (s[:-1] >= 0)).any())


def split_inner(idx: np.ndarray) -> int:
    """Number of trailing position axes along which ``idx (k, *s)`` is constant.  Tables
    are stored without those axes, so consecutive threads share one table entry."""
    n_inner = 0
    for ax in range(idx.ndim - 1, 0, -1):
        first = np.take(idx, [0], axis=ax)
        if idx.shape[ax] == 1 or (idx == first).all():
            idx = first
            n_inner += 1
        else:
            break
    return n_inner


def per_position_sorted_unique(arr: np.ndarray) -> np.ndarray:
    """Sorted unique non-negative values along the last axis, ``-1`` padded at the end;
    width = the largest per-position count (folx/hessian.py:234-258)."""
    lead = arr.shape[:-1]
    if arr.shape[-1] == 0:
        return np.full((*lead, 0), -1, dtype=arr.dtype)
    s = np.sort(arr, axis=-1)
    prev = np.concatenate([np.full((*lead, 1), -2, dtype=arr.dtype), s[..., :-1]], axis=-1)
    first = (s != prev) & (s >= 0)
    big = np.iinfo(arr.dtype).max
    packed = np.sort(np.where(first, s, big), axis=-1)
    width = int(first.sum(-1).max()) if first.size else 0
    out = packed[..., :width]
    return np.where(out == big, -1, out)


def per_position_intersection(masks: Sequence[np.ndarray]) -> np.ndarray:
    """Values present in every operand's set, per position (folx/hessian.py:261-285)."""
    n = len(masks)
    per = [per_position_sorted_unique(m) for m in masks]
    comb = np.concatenate(per, axis=-1)
    lead, total = comb.shape[:-1], comb.shape[-1]
    if total < n:
        return np.full((*lead, 0), -1, dtype=comb.dtype)
    s = np.sort(comb, axis=-1)
    first, last = s[..., : total - n + 1], s[..., n - 1 :]
    hit = (first == last) & (first >= 0)
    big = np.iinfo(comb.dtype).max
    packed = np.sort(np.where(hit, first, big), axis=-1)
    width = int(hit.sum(-1).max()) if hit.size else 0
    out = packed[..., :width]
    return np.where(out == big, -1, out)


# --------------------------------------------------------------------------------------
# row re-indexing
# --------------------------------------------------------------------------------------


def get_index_mask(mask: np.ndarray, outputs: np.ndarray) -> np.ndarray:
    """Slot of ``outputs`` (axis 0) holding the same input index as each sparse entry, or
    ``-1``; first match wins (folx/api.py:120-159)."""
    s = np.broadcast_shapes(mask.shape[1:], outputs.shape[1:])
    m = np.broadcast_to(mask, (mask.shape[0], *s))
    if outputs.shape[0] == 0:
        return np.full(m.shape, -1, dtype=INT)
    o = np.broadcast_to(outputs, (outputs.shape[0], *s))
    match = m[:, None] == o[None]  # (k, T, *s)
    idx = match.argmax(1)
    return np.where(match.any(1), idx, -1).astype(INT)


def gather_table(idx: np.ndarray, n_out: int):
    """Static gather table of ``materialize_by_gather`` (folx/utils.py:71-114).

    idx (k, *s): target row of every source entry, ``-1`` = none.
    Returns ``take (n_out, n_slots, *s)`` int32: the source rows summed into target row t
    at each position, ``-1`` padded; sources keep their original order within a target
    (stable sort), which fixes the floating-point summation order.
    """
    k = idx.shape[0]
    s = idx.shape[1:]
    S = int(np.prod(s, dtype=int))
    flat = idx.reshape(k, S).T  # (S, k)
    if k == 0 or S == 0:
        return np.full((n_out, 1, *s), -1, dtype=np.int32)
    order = np.argsort(flat, axis=1, kind='stable')
    st = np.take_along_axis(flat, order, axis=1)
    first = np.concatenate([np.ones((S, 1), dtype=bool), st[:, 1:] != st[:, :-1]], axis=1)
    ar = np.arange(k)[None, :]
    run_start = np.maximum.accumulate(np.where(first, ar, 0), axis=1)
    slot = ar - run_start
    valid = st >= 0
    n_slots = int(slot[valid].max()) + 1 if valid.any() else 1
    take = np.full((S, n_out, n_slots), -1, dtype=np.int32)
    pos = np.broadcast_to(np.arange(S)[:, None], (S, k))
    take[pos[valid], st[valid], slot[valid]] = order[valid]
    return np.ascontiguousarray(np.moveaxis(take, 0, -1)).reshape(n_out, n_slots, *s)


def reduction_frame(masks: Sequence[np.ndarray], axes) -> np.ndarray:
    """Index part of ``get_jacobian_for_reduction`` (folx/utils.py:499-588): per kept
    position, the ascending union of valid indices over all operands, rows and reduced
    axes, ``-1`` padded at the END.  Returns ``(m, *kept_shape)``."""
    s = np.broadcast_shapes(*[m.shape[1:] for m in masks])
    nd = len(s)
    axes = tuple(sorted(a % nd for a in np.atleast_1d(axes)))
    kept = [a for a in range(nd) if a not in axes]
    cols = []
    for m in masks:
        m = np.broadcast_to(m, (m.shape[0], *s))
        m = np.transpose(m, [a + 1 for a in kept] + [0] + [a + 1 for a in axes])
        cols.append(m.reshape(*[s[a] for a in kept], -1))
    allv = np.concatenate(cols, axis=-1).astype(INT)
    out = per_position_sorted_unique(allv)
    return np.moveaxis(out, -1, 0)


@_memo
def sum_out_mask(mask: np.ndarray, axes):
    """Index part of ``sparse_sum_jvp`` (folx/jvp.py:108-146).

    Per output position the distinct values over rows and reduced axes, ascending, with
    ``-1`` treated as a value (so it sorts FIRST, :116-126), ``-1`` filled at the end.
    Returns ``(idx_out (m, *kept), slot (k, *s))``; ``slot`` is the output row each input
    entry is summed into (first match, :144).
    """
    k, *s = mask.shape
    nd = len(s)
    axes = tuple(sorted(a % nd for a in np.atleast_1d(axes)))
    kept = [a for a in range(nd) if a not in axes]
    perm = [a + 1 for a in kept] + [0] + [a + 1 for a in axes]
    m = np.transpose(mask, perm).astype(INT)
    kept_shape = [s[a] for a in kept]
    flat = m.reshape(*kept_shape, -1)  # (*kept, k * red)
    srt = np.sort(flat, axis=-1)
    prev = np.concatenate(
        [np.full((*kept_shape, 1), np.iinfo(INT).min, dtype=INT), srt[..., :-1]], axis=-1
    )
    first = srt != prev
    width = int(first.sum(-1).max())
    big = np.iinfo(INT).max
    packed = np.sort(np.where(first, srt, big), axis=-1)[..., :width]
    idx_out = np.where(packed == big, -1, packed)  # (*kept, width)
    match = flat[..., :, None] == idx_out[..., None, :]  # (*kept, k*red, width)
    slot_flat = match.argmax(-1)
    slot = slot_flat.reshape(*kept_shape, k, *[s[a] for a in axes])
    slot = np.transpose(slot, np.argsort(perm))
    return np.moveaxis(idx_out, -1, 0), slot


@_memo
def rows_distinct(mask: np.ndarray) -> bool:
    """No two rows of the mask are the same over all positions."""
    k = mask.shape[0]
    flat = np.ascontiguousarray(mask).reshape(k, -1)
    return all(not np.array_equal(flat[i], flat[j]) for i in range(k) for j in range(i))


@_memo
def merge_rows(masks: Sequence[np.ndarray]):
    """Row merge of a multi-operand elementwise op (folx/jvp.py:294-317): broadcast and
    concatenate the masks along the row axis, merge identical rows with
    ``np.unique(axis=0)``.  Returns ``(result_mask, inverse)``."""
    s = np.broadcast_shapes(*[m.shape[1:] for m in masks])
    cat = np.concatenate([np.broadcast_to(m, (m.shape[0], *s)) for m in masks], axis=0)
    res, inv = np.unique(cat, axis=0, return_inverse=True)
    return res, np.asarray(inv).reshape(-1)


def find_out_idx(masks, x_shapes, in_axes, linear_in_one: bool, threshold: int):
    """``hessian.find_out_idx`` (folx/hessian.py:288-340).

    masks[i] is ``(k_i, *x_shapes[i])`` (pass ``FwdJacobian.mask`` for dense operands) or
    None for all-dense calls.  ``in_axes[i]`` are the axes operand i is consumed along.
    The position frame is the broadcast of the operands' remaining axes with the axes that
    have size 1 in every operand dropped (folx/utils.py:271-327).  Returns
    ``(idx (M, *frame), dense_out)``.
    """
    if all(m is None for m in masks):
        return None, True
    n_args = len(masks)
    pos_shapes, perms = [], []
    for m, xs, ax in zip(masks, x_shapes, in_axes):
        nd = len(xs)
        axn = tuple(a % nd for a in ax) if nd else ()
        mapped = [a for a in range(nd) if a not in axn]
        pos_shapes.append([xs[a] for a in mapped])
        perms.append((mapped, [a for a in range(nd) if a in axn]))
    nfr = max(len(p) for p in pos_shapes)
    padded = [[1] * (nfr - len(p)) + list(p) for p in pos_shapes]
    keep = [d for d in range(nfr) if any(p[d] != 1 for p in padded)]
    frame = [max(p[d] for p in padded) for d in keep]

    aligned = []
    for m, xs, (mapped, red), pp in zip(masks, x_shapes, perms, padded):
        m = np.asarray(m).astype(INT)
        # (mapped axes..., row axis, consumed axes...) -> (*padded frame, K_flat)
        t = np.transpose(m, [a + 1 for a in mapped] + [0] + [a + 1 for a in red])
        t = t.reshape(*pp, -1)
        t = t.reshape(*[pp[d] for d in keep], t.shape[-1])  # dropped dims have size 1
        aligned.append(np.broadcast_to(t, (*frame, t.shape[-1])))

    max_size = max(int((np.unique(np.asarray(m)) >= 0).sum()) for m in masks)
    if linear_in_one:
        idx = per_position_intersection(aligned)
    else:
        idx = per_position_sorted_unique(np.concatenate(aligned, axis=-1))
    idx = np.moveaxis(idx, -1, 0)
    dense_out = bool(idx.shape[0] >= max_size or idx.shape[0] > threshold)
    return idx, dense_out


@_memo
def dot_projection(mask: np.ndarray, contract_axis: int, threshold: int):
    """Mask of ``h @ W`` for sparse ``h`` with one contracted axis
    (folx/wrapped_functions.py:113-157).  Returns ``(proj, aligned)``: ``proj`` is
    ``(k', *s_without_contract, 1)`` -- rows unchanged when the mask is constant along the
    contracted axis (:131-133), else the union frame (``aligned`` True), or None when
    that union exceeds the threshold (:129-130)."""
    nd = mask.ndim - 1
    ca = contract_axis % nd
    first = np.take(mask, [0], axis=ca + 1)
    if (mask == first).all():
        return np.take(mask, 0, axis=ca + 1)[..., None], False
    proj = reduction_frame([mask], (ca,))
    if proj.shape[0] > threshold:
        return None, True
    return proj[..., None], True


# --------------------------------------------------------------------------------------
# sparse slogdet planner (folx/slogdet.py:73-293)
# --------------------------------------------------------------------------------------

SLOGDET_MAX_MASK_ENTRIES = 2**24  # bound of the host-side mask analysis (folx/slogdet.py:73)


def slogdet_entry_mask(x0_idx, k: int, x_shape, transposed: bool):
    """Mask ``(k, n, m)`` naming the input coordinate of every (stored row, matrix row,
    column) entry, if it is the same for every batch position; else None
    (``_entry_mask``, folx/slogdet.py:94-125).  ``transposed`` describes A^T."""
    if x0_idx is None:
        return None
    idx = np.asarray(x0_idx)
    shape = tuple(int(d) for d in x_shape)
    if transposed:
        if idx.ndim != len(shape) + 1:
            return None
        idx = idx.swapaxes(-1, -2)
        shape = shape[:-2] + (shape[-1], shape[-2])
    if k * int(np.prod(shape, dtype=np.int64)) > SLOGDET_MAX_MASK_ENTRIES:
        return None
    n, m = shape[-2:]
    full = np.broadcast_to(idx, (k, *shape)).reshape(k, -1, n, m)
    if not (full == full[:, :1]).all():
        return None
    return np.ascontiguousarray(full[:, 0]).astype(INT)


def _rank_in_group(sorted_keys: np.ndarray) -> np.ndarray:
    """Position of every element inside its run of equal (sorted) keys."""
    return np.arange(sorted_keys.size) - np.searchsorted(sorted_keys, sorted_keys, side='left')


def slogdet_factor_tables(mask: np.ndarray, per_entry: bool):
    """Static tables that split every ``dA/dx_c`` into rank-one factors: one per touched
    row, or one per touched entry with ``per_entry`` (``_factor_tables``,
    folx/slogdet.py:142-179).  Returns ``(cost, tables)`` or None when the tables would
    be too large; ``tables``: ``take (C, rank, width)`` flat (stored row, row, column)
    addresses with ``k n m`` for unused slots, ``cols`` likewise, ``rows (C, rank)``,
    ``coords (C,)``, ``per_entry``."""
    k, n, m = mask.shape
    flat = mask.reshape(-1)
    pos = np.flatnonzero(flat >= 0)
    coords, ci = np.unique(flat[pos], return_inverse=True)
    ci = ci.reshape(-1)
    r, c = np.divmod(pos % (n * m), m)
    fkey = (ci * n + r) * m + (c if per_entry else 0)
    # entries ordered by factor, then column, then stored row (pos is ascending in the latter)
    order = np.lexsort((pos, c, fkey))
    pos, c, fkey = pos[order], c[order], fkey[order]
    fkeys, f_of = np.unique(fkey, return_inverse=True)
    f_of = f_of.reshape(-1)
    f_coord = fkeys // (n * m)
    slot = _rank_in_group(f_coord)
    within = _rank_in_group(fkey)
    rank, width = int(slot.max()) + 1, int(within.max()) + 1
    C = coords.size
    if C * rank * width > SLOGDET_MAX_MASK_ENTRIES:
        return None
    take = np.full((C, rank, width), k * n * m, dtype=INT)
    cols = np.zeros((C, rank, width), dtype=INT)
    rows = np.zeros((C, rank), dtype=INT)
    take[f_coord[f_of], slot[f_of], within] = pos
    cols[f_coord[f_of], slot[f_of], within] = c
    rows[f_coord, slot] = (fkeys % (n * m)) // m
    cost = C * rank * rank * (1 if per_entry else width)
    return cost, dict(take=take, cols=cols, rows=rows, coords=coords.astype(INT), per_entry=per_entry)


def slogdet_plan(x0_idx, k: int, x_shape, max_n: int):
    """Cheapest of the four decompositions (rows or entries of A, rows of A^T; the first
    of equal costs wins), if it beats contracting the dense Jacobian (``sparse_slogdet``,
    folx/slogdet.py:249-293).  Returns ``(tables, transposed)`` or None."""
    best = None
    for transposed in (False, True):
        mask = slogdet_entry_mask(x0_idx, k, x_shape, transposed)
        if mask is None or not (mask >= 0).any():
            continue
        for per_entry in ((False,) if transposed else (False, True)):
            plan = slogdet_factor_tables(mask, per_entry)
            if plan is not None and (best is None or plan[0] < best[0]):
                best = (plan[0], plan[1], transposed)
    if best is None:
        return None
    cost, tables, transposed = best
    n, m = x_shape[-2:]
    tangents = max_n + 1
    if 4 * cost > tangents * n * m * (n + 1) or cost > 2 * tangents * n * m:
        return None
    return tables, transposed


def slogdet_kernel_tables(tables, transposed: bool, k: int, n: int):
    """int32 tables in the kernel's convention: ``take`` addresses the Jacobian as stored
    (for tables of A^T the row and column of every address are swapped back) and unused
    slots are ``-1``."""
    take = tables['take']
    valid = take < k * n * n
    t, rem = np.divmod(np.where(valid, take, 0), n * n)
    r, c = np.divmod(rem, n)
    addr = (t * n + c) * n + r if transposed else (t * n + r) * n + c
    take32 = np.where(valid, addr, -1).astype(np.int32)
    return take32, tables['cols'].astype(np.int32), tables['rows'].astype(np.int32)


# --------------------------------------------------------------------------------------
# static positions of indexed reads and scatters (folx/jvp.py:416-471, :536-609)
# --------------------------------------------------------------------------------------


def index_positions(shape, idx) -> np.ndarray:
    """Flat position in an array of ``shape`` that every element of ``array[idx]`` refers
    to, for a static numpy index (ints, slices, ``None``, ``Ellipsis``, integer arrays).
    Integer-array entries outside ``[-size, size)`` give ``-1`` (a scatter drops those
    updates, folx/jvp.py:434-435); negative ones count from the end."""
    shape = tuple(int(d) for d in shape)
    idx = idx if isinstance(idx, tuple) else (idx,)
    n_named = sum(1 for i in idx if i is not None and i is not Ellipsis)
    assert n_named <= len(shape), 'too many indices'
    # walk the index to find the axis every integer array applies to
    axis, padded_axes, new_idx = 0, [], []
    for i in idx:
        if i is None:
            new_idx.append(None)
        elif i is Ellipsis:
            axis += len(shape) - n_named
            new_idx.append(Ellipsis)
        elif isinstance(i, (slice, int, np.integer)):
            new_idx.append(i)
            axis += 1
        else:
            arr = np.asarray(i)
            assert arr.dtype.kind in 'iu', 'only integer index arrays are static positions'
            size = shape[axis]
            arr = np.where(arr < 0, arr + size, arr)
            # out-of-range entries point at an extra slot that holds -1
            new_idx.append(np.where((arr < 0) | (arr >= size), size, arr))
            padded_axes.append(axis)
            axis += 1
    pos = np.arange(int(np.prod(shape, dtype=np.int64)), dtype=INT).reshape(shape)
    for ax in padded_axes:
        pad = [(0, 0)] * len(shape)
        pad[ax] = (0, 1)
        pos = np.pad(pos, pad, constant_values=-1)
    return np.asarray(pos[tuple(new_idx)])


def scatter_source_table(tpos: np.ndarray, op_size: int, last_only: bool) -> np.ndarray:
    """For every operand position the update elements that land on it, ascending, ``-1``
    padded: ``(op_size, n_slots)`` int32 (at least one slot).  ``last_only`` keeps the last
    element only (a 'set' is decided by the final write)."""
    t = np.asarray(tpos).reshape(-1)
    e = np.flatnonzero(t >= 0)
    p = t[e]
    order = np.argsort(p, kind='stable')
    p, e = p[order], e[order]
    slot = np.arange(p.size) - np.searchsorted(p, p, side='left')
    if last_only and p.size:
        count = np.bincount(p, minlength=op_size)
        keep = slot == count[p] - 1
        p, e, slot = p[keep], e[keep], np.zeros(int(keep.sum()), dtype=INT)
    n_slots = int(slot.max()) + 1 if p.size else 1
    table = np.full((op_size, n_slots), -1, dtype=np.int32)
    table[p, slot] = e
    return table


def scatter_out_mask(op_mask, upd_mask, tpos: np.ndarray, op_shape, is_set: bool) -> np.ndarray:
    """Mask of a scatter's output (folx/jvp.py:536-609): per operand position the ascending
    union of the operand's dependencies (none where a 'set' overwrites the position) and of
    those of the update elements landing there, ``-1`` padded at the end; at least one row."""
    op_shape = tuple(int(d) for d in op_shape)
    op_size = int(np.prod(op_shape, dtype=np.int64))
    tflat = np.asarray(tpos).reshape(-1)
    pos_parts, dep_parts = [], []
    if upd_mask is not None:
        um = np.broadcast_to(upd_mask, (upd_mask.shape[0], *np.shape(tpos))).reshape(upd_mask.shape[0], -1)
        tp = np.broadcast_to(tflat, um.shape)
        sel = (um >= 0) & (tp >= 0)
        pos_parts.append(tp[sel]), dep_parts.append(um[sel])
    if op_mask is not None:
        om = np.broadcast_to(op_mask, (op_mask.shape[0], *op_shape)).reshape(op_mask.shape[0], -1)
        keep = om >= 0
        if is_set:
            hit = np.zeros(op_size, dtype=bool)
            hit[tflat[tflat >= 0]] = True
            keep = keep & ~hit
        pp = np.broadcast_to(np.arange(op_size), om.shape)
        pos_parts.append(pp[keep]), dep_parts.append(om[keep])
    pos = np.concatenate(pos_parts).astype(INT) if pos_parts else np.zeros(0, INT)
    dep = np.concatenate(dep_parts).astype(INT) if dep_parts else np.zeros(0, INT)
    if pos.size == 0:
        return np.full((1, *op_shape), -1, dtype=np.int32)
    span = int(dep.max()) + 1
    keys = np.unique(pos * span + dep)   # sorted by position, then dependency
    kp, kd = keys // span, keys % span
    slot = np.arange(kp.size) - np.searchsorted(kp, kp, side='left')
    out = np.full((int(slot.max()) + 1, op_size), -1, dtype=np.int32)
    out[slot, kp] = kd
    return out.reshape(out.shape[0], *op_shape)

"""Integer restatement of the reference's static sparsity algebra (test infrastructure).

A sparse Jacobian stores ``k`` rows ``data (k, *s)`` and a host-side int mask
``x0_idx (k, *s)`` naming the input coordinate each entry differentiates against, ``-1``
for "no entry" (folx/api.py:19-42).  Everything here is written as explicit loops over
positions so that it is an independent check of the vectorised host code in the product.
"""

from __future__ import annotations

import itertools

import numpy as np


def dense_mask(P: int, shape) -> np.ndarray:
    """Mask of a dense Jacobian: row p depends on input p (folx/api.py:211-220)."""
    m = np.arange(P, dtype=np.int64).reshape(P, *([1] * len(shape)))
    return np.broadcast_to(m, (P, *shape)).copy()


def init_mask(shape) -> np.ndarray:
    """Initial sparse mask: one row, entry i depends on flat input i
    (folx/interpreter.py:283-293)."""
    n = int(np.prod(shape, dtype=int))
    return np.arange(n, dtype=np.int64).reshape(1, *shape)


def materialize(data: np.ndarray, idx: np.ndarray, n_out: int) -> np.ndarray:
    """out[t, pos] = sum of data[r, pos] over rows r with idx[r, pos] == t.

    Semantics of ``FwdJacobian.materialize_for_idx`` (folx/api.py:58-118) whose two
    implementations (static gather table folx/utils.py:71-114, ``segment_sum``
    folx/api.py:110-114) both compute this sum; rows with idx < 0 map nowhere.
    ``data`` may carry extra axes between the row axis and the position axes that the
    mask does not have (the walker axis): data (k, B, *s), idx (k, *s).
    """
    k = idx.shape[0]
    s = idx.shape[1:]
    extra = data.ndim - idx.ndim
    lead = data.shape[1 : 1 + extra]
    out = np.zeros((n_out, *lead, *s), dtype=data.dtype)
    for r in range(k):
        for pos in itertools.product(*[range(n) for n in s]):
            t = int(idx[(r, *pos)])
            if t >= 0:
                sl = (slice(None),) * extra
                out[(t, *sl, *pos)] += data[(r, *sl, *pos)]
    return out


def get_index_mask(mask: np.ndarray, outputs: np.ndarray) -> np.ndarray:
    """For every sparse row entry, the slot of ``outputs`` (axis 0) holding the same
    input index at that position, or -1 (folx/api.py:120-159: first match via argmax).
    ``mask`` (k, *s) and ``outputs`` (T, *s') broadcast against each other on the
    position axes."""
    s = np.broadcast_shapes(mask.shape[1:], outputs.shape[1:])
    mask = np.broadcast_to(mask, (mask.shape[0], *s))
    outputs = np.broadcast_to(outputs, (outputs.shape[0], *s))
    res = np.full(mask.shape, -1, dtype=np.int64)
    for pos in itertools.product(*[range(n) for n in s]):
        col = outputs[(slice(None), *pos)]
        for r in range(mask.shape[0]):
            hits = np.nonzero(col == mask[(r, *pos)])[0]
            if hits.size:
                res[(r, *pos)] = hits[0]
    return res


def dense_array(data: np.ndarray, mask: np.ndarray) -> np.ndarray:
    """``FwdJacobian.dense_array`` for a sparse Jacobian: rows 0..max(mask)
    (folx/api.py:182-190, :192-196)."""
    n_out = int(mask.max()) + 1
    return materialize(data, mask, n_out)


def has_duplicates(mask: np.ndarray | None) -> bool:
    """True iff some position lists a valid index twice (folx/hessian.py:71-84)."""
    if mask is None or mask.shape[0] <= 1:
        return False
    s = mask.shape[1:]
    for pos in itertools.product(*[range(n) for n in s]):
        col = [int(v) for v in mask[(slice(None), *pos)] if v >= 0]
        if len(col) != len(set(col)):
            return True
    return False


def _pad_columns(cols, pad_at_end=True):
    m = max((len(c) for c in cols), default=0)
    return [list(c) + [-1] * (m - len(c)) for c in cols], m


def reduction_frame(masks, axes):
    """Index part of ``get_jacobian_for_reduction`` (folx/utils.py:499-588).

    For every kept (non-reduced) position: the sorted union, over all operands, all rows
    and all reduced axes, of the valid input indices; ``-1`` entries are dropped and the
    lists are padded with ``-1`` at the END (:557-566).  Returns ``(max_unique, *kept)``.
    ``masks``: sequence of (k_i, *s) arrays broadcastable on the position axes.
    """
    s = np.broadcast_shapes(*[m.shape[1:] for m in masks])
    masks = [np.broadcast_to(m, (m.shape[0], *s)) for m in masks]
    nd = len(s)
    axes = tuple(a % nd for a in np.atleast_1d(axes))
    kept = [a for a in range(nd) if a not in axes]
    kept_shape = [s[a] for a in kept]
    cols = []
    for pos in itertools.product(*[range(n) for n in kept_shape]):
        vals = set()
        for m in masks:
            index = [slice(None)] * (nd + 1)
            for a, p in zip(kept, pos):
                index[a + 1] = p
            sub = m[tuple(index)]
            vals.update(int(v) for v in sub.reshape(-1) if v != -1)
        cols.append(sorted(vals))
    cols, m = _pad_columns(cols)
    out = np.array(cols, dtype=np.int64).reshape(*kept_shape, m)
    return np.moveaxis(out, -1, 0)


def sum_out_mask(mask: np.ndarray, axes):
    """Index part of ``sparse_sum_jvp`` (folx/jvp.py:108-146).

    Per output position, the distinct values found over the rows and the reduced axes,
    ascending -- ``-1`` counts as a value and therefore sorts FIRST (:116-126) -- padded
    at the end with ``-1``.  Returns ``(idx_out (m, *out_shape), slot (k, *s))`` where
    ``slot`` is the output row every input entry is summed into (:144, first match).
    """
    k, *s = mask.shape
    nd = len(s)
    axes = tuple(a % nd for a in np.atleast_1d(axes))
    kept = [a for a in range(nd) if a not in axes]
    kept_shape = [s[a] for a in kept]
    cols = {}
    for pos in itertools.product(*[range(n) for n in kept_shape]):
        index = [slice(None)] * (nd + 1)
        for a, p in zip(kept, pos):
            index[a + 1] = p
        sub = mask[tuple(index)]
        cols[pos] = sorted(set(int(v) for v in sub.reshape(-1)))
    m = max(len(c) for c in cols.values())
    idx_out = np.full((m, *kept_shape), -1, dtype=np.int64)
    for pos, c in cols.items():
        idx_out[(slice(0, len(c)), *pos)] = c
    slot = np.zeros(mask.shape, dtype=np.int64)
    for full in itertools.product(*[range(n) for n in mask.shape]):
        pos = tuple(full[1 + a] for a in kept)
        col = idx_out[(slice(None), *pos)]
        slot[full] = int(np.nonzero(col == mask[full])[0][0])
    return idx_out, slot


def merge_binary_masks(masks):
    """Row merge of a multi-operand elementwise op (folx/jvp.py:294-317): the operands'
    masks are broadcast and concatenated along the row axis, identical rows are merged by
    ``np.unique(axis=0)`` (lexicographic row order).  Returns ``(result_mask, inverse)``
    where ``inverse[r]`` is the output row that concatenated input row ``r`` adds into."""
    s = np.broadcast_shapes(*[m.shape[1:] for m in masks])
    cat = np.concatenate(
        [np.broadcast_to(m, (m.shape[0], *s)) for m in masks], axis=0
    )
    flat = cat.reshape(cat.shape[0], -1)
    uniq = sorted(set(tuple(int(v) for v in row) for row in flat))
    inverse = np.array([uniq.index(tuple(int(v) for v in row)) for row in flat])
    result = np.array(uniq, dtype=np.int64).reshape(len(uniq), *s)
    return result, inverse


def add_masks(mask_a, mask_b):
    """``FwdJacobian.__add__`` for two sparse Jacobians (folx/api.py:230-249): equal masks
    add in place (returns ``('same', mask)``), different masks concatenate rows."""
    if mask_a.shape[0] == mask_b.shape[0] and np.array_equal(
        *np.broadcast_arrays(mask_a, mask_b)
    ):
        return 'same', np.broadcast_arrays(mask_a, mask_b)[0]
    return 'concat', np.concatenate([mask_a, mask_b], axis=0)


def find_out_idx(masks, x_shapes, in_axes, linear_in_one: bool, threshold: int):
    """``hessian.find_out_idx`` (folx/hessian.py:288-340).

    masks[i]    : (k_i, *x_shapes[i]) int mask, or None for a dense Jacobian whose row
                  count is given by ``x_shapes[i]`` being paired with ``dense_rows[i]``
                  -- dense operands are passed as explicit ``dense_mask`` arrays instead.
    in_axes[i]  : the axes of operand i that the function consumes jointly (not mapped).
    Returns ``(idx, dense_out)``; ``idx`` is ``(M, *frame)`` where ``frame`` is the
    broadcast of the operands' mapped axes with all-size-1 axes dropped (:312-322 via
    folx/utils.py:271-327), union of valid indices per position or intersection when
    ``linear_in_one`` (:331-334), ascending, ``-1`` padded at the end (:234-285).
    ``dense_out`` is True when M >= the largest per-operand count of distinct valid
    indices, or M > threshold (:338-340).
    """
    if all(m is None for m in masks):
        return None, True
    pos_shapes = []
    for m, xs, ax in zip(masks, x_shapes, in_axes):
        nd = len(xs)
        ax = tuple(a % nd for a in ax) if nd else ()
        pos_shapes.append([xs[a] for a in range(nd) if a not in ax])
    nfr = max(len(p) for p in pos_shapes)
    padded = [[1] * (nfr - len(p)) + p for p in pos_shapes]
    frame = [max(p[d] for p in padded) for d in range(nfr)]
    keep = [d for d in range(nfr) if any(p[d] != 1 for p in padded)]
    out_frame = [frame[d] for d in keep]

    max_size = 0
    for m in masks:
        u = np.unique(m)
        max_size = max(max_size, int((u >= 0).sum()))

    cols = []
    for pos in itertools.product(*[range(frame[d]) for d in keep]):
        full_pos = [0] * nfr
        for d, p in zip(keep, pos):
            full_pos[d] = p
        sets = []
        for m, xs, ax, pp in zip(masks, x_shapes, in_axes, padded):
            nd = len(xs)
            axn = tuple(a % nd for a in ax) if nd else ()
            mapped = [a for a in range(nd) if a not in axn]
            index = [slice(None)] * (nd + 1)
            off = nfr - len(mapped)
            for j, a in enumerate(mapped):
                index[a + 1] = full_pos[off + j] if xs[a] != 1 else 0
            sub = m[tuple(index)]
            sets.append(set(int(v) for v in sub.reshape(-1) if v >= 0))
        if linear_in_one:
            vals = set.intersection(*sets)
        else:
            vals = set.union(*sets)
        cols.append(sorted(vals))
    cols, M = _pad_columns(cols)
    idx = np.array(cols, dtype=np.int64).reshape(*out_frame, M)
    idx = np.moveaxis(idx, -1, 0)
    dense_out = bool(M >= max_size or M > threshold)
    return idx, dense_out


def dot_projection(mask: np.ndarray, contract_axis: int, threshold: int):
    """Mask of ``h @ W`` for a sparse ``h`` (folx/wrapped_functions.py:113-157), for a
    single contracted axis of ``h`` and a constant ``W`` with one new output axis that
    takes the contracted axis' place at the end.

    If the mask is constant along the contracted axis the rows pass through unchanged
    (index 0 taken, :131-133); otherwise rows are aligned to the per-position union
    (``reduction_frame``) and the result is None when that union exceeds the threshold
    (:129-130).  Returns ``(proj (k', *s_without_contract, 1), aligned: bool)``.
    """
    nd = mask.ndim - 1
    ca = contract_axis % nd
    first = np.take(mask, [0], axis=ca + 1)
    if np.array_equal(mask, np.broadcast_to(first, mask.shape)):
        proj = np.take(mask, 0, axis=ca + 1)
        return proj[..., None], False
    proj = reduction_frame([mask], (ca,))
    if proj.shape[0] > threshold:
        return None, True
    return proj[..., None], True


# --------------------------------------------------------------------------------------
# Sparse slogdet planner (folx/slogdet.py:73-293)
# --------------------------------------------------------------------------------------

SLOGDET_MAX_MASK_ENTRIES = 2**24  # folx/slogdet.py:73


def slogdet_entry_mask(x0_idx, k: int, x_shape, transposed: bool):
    """Per-entry coordinate mask ``(k, n, m)`` shared by all batch positions, or None
    (folx/slogdet.py:94-125).  ``x_shape`` is the per-walker shape ``(..., n, m)`` of the
    matrix array, ``k`` the number of stored Jacobian rows."""
    if x0_idx is None:
        return None
    idx = np.asarray(x0_idx)
    shape = tuple(x_shape)
    if transposed:
        if idx.ndim != len(shape) + 1:
            return None
        idx = np.swapaxes(idx, -1, -2)
        shape = (*shape[:-2], shape[-1], shape[-2])
    if k * int(np.prod(shape, dtype=np.int64)) > SLOGDET_MAX_MASK_ENTRIES:
        return None
    full = np.broadcast_to(idx, (k, *shape))
    n, m = shape[-2:]
    first = None
    for pos in itertools.product(*[range(d) for d in shape[:-2]]):
        cur = full[(slice(None), *pos)]
        if first is None:
            first = cur
        elif not np.array_equal(first, cur):
            return None
    return np.ascontiguousarray(first).astype(np.int64).reshape(k, n, m)


def slogdet_factor_tables(mask: np.ndarray, per_entry: bool):
    """Rank-one factor tables of every ``dA/dx_c`` (folx/slogdet.py:142-179).

    A factor is one touched row of ``dA/dx_c`` (or one touched entry with ``per_entry``).
    Returns ``(cost, tables)`` with ``tables`` a dict: ``take (C, rank, width)`` flat
    ``(tangent, row, column)`` addresses (``k n m`` = unused), ``cols (C, rank, width)``,
    ``rows (C, rank)``, ``coords (C,)``, ``per_entry``; None when the tables are too large.
    """
    k, n, m = mask.shape
    by_coord: dict[int, list] = {}
    for t in range(k):
        for r in range(n):
            for c in range(m):
                v = int(mask[t, r, c])
                if v >= 0:
                    by_coord.setdefault(v, []).append((r, c, t))
    coords = sorted(by_coord)
    factor_lists = []
    for v in coords:
        entries = sorted(by_coord[v])  # by row, column, then tangent
        factors: dict[tuple, list] = {}
        for r, c, t in entries:
            key = (r, c) if per_entry else (r,)
            factors.setdefault(key, []).append((r, c, t))
        factor_lists.append([factors[key] for key in sorted(factors)])
    rank = max(len(f) for f in factor_lists)
    width = max(len(e) for f in factor_lists for e in f)
    C = len(coords)
    if C * rank * width > SLOGDET_MAX_MASK_ENTRIES:
        return None
    take = np.full((C, rank, width), k * n * m, dtype=np.int64)
    cols = np.zeros((C, rank, width), dtype=np.int64)
    rows = np.zeros((C, rank), dtype=np.int64)
    for ci, facs in enumerate(factor_lists):
        for s, ents in enumerate(facs):
            rows[ci, s] = ents[0][0]
            for l, (r, c, t) in enumerate(ents):
                take[ci, s, l] = (t * n + r) * m + c
                cols[ci, s, l] = c
    cost = C * rank * rank * (1 if per_entry else width)
    return cost, dict(take=take, cols=cols, rows=rows, coords=np.asarray(coords, dtype=np.int64),
                      per_entry=per_entry)


def slogdet_plan(x0_idx, k: int, x_shape, max_n: int):
    """Choice among the four decompositions and the gate against the dense contraction
    (folx/slogdet.py:249-293).  Returns ``(tables, transposed)`` or None."""
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


# --------------------------------------------------------------------------------------
# Scatter (folx/jvp.py:474-673)
# --------------------------------------------------------------------------------------


def scatter_out_mask(op_mask, upd_mask, tpos, op_shape, is_set: bool):
    """Output mask of a scatter with static target positions (folx/jvp.py:536-609): per
    operand position the ascending union of the operand's dependencies (dropped where a
    'set' overwrites the position, :549-553) and of the dependencies of every update
    element landing there; ``-1`` padded at the end, at least one row.

    op_mask (k_op, *op_shape) or None (constant operand), upd_mask (k_upd, *upd_shape) or
    None, tpos (*upd_shape) flat operand positions (-1 = dropped)."""
    op_size = int(np.prod(op_shape, dtype=int))
    tflat = np.asarray(tpos).reshape(-1)
    deps = [set() for _ in range(op_size)]
    overwritten = set(int(p) for p in tflat if p >= 0)
    if op_mask is not None:
        om = np.broadcast_to(op_mask, (op_mask.shape[0], *op_shape)).reshape(op_mask.shape[0], -1)
        for p in range(op_size):
            if is_set and p in overwritten:
                continue
            deps[p] |= {int(v) for v in om[:, p] if v >= 0}
    if upd_mask is not None:
        um = np.broadcast_to(upd_mask, (upd_mask.shape[0], *np.shape(tpos))).reshape(upd_mask.shape[0], -1)
        for e, p in enumerate(tflat):
            if p >= 0:
                deps[int(p)] |= {int(v) for v in um[:, e] if v >= 0}
    max_out = max(1, max((len(d) for d in deps), default=0))
    out = np.full((max_out, op_size), -1, dtype=np.int64)
    for p, d in enumerate(deps):
        for r, v in enumerate(sorted(d)):
            out[r, p] = v
    return out.reshape(max_out, *op_shape)

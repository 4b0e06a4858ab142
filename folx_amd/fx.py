"""A traced front door: ``forward_laplacian_torch(fn, sparsity_threshold)`` takes a model written with PLAIN TORCH
(one sample in, tensors out), traces it once per input shape into a graph of primitive operations and evaluates
that graph equation by equation through the rule registry -- what the reference does with a jaxpr
(``eval_jaxpr_with_forward_laplacian``, folx/interpreter.py:127-264: per equation, constants are evaluated
eagerly (:222-245), everything else looks its rule up under the primitive's name (:210-216), a primitive
without a rule gets the generic wrap with a warning, folx/wrapped_functions.py:597-618).

Here the trace is ``torch.fx`` (``make_fx`` on a CPU example: an ATen-level graph with concrete shapes, module
parameters lifted to graph constants) and an equation's rule is the ``folx_amd.numpy`` function of the same
meaning, which dispatches to the registry under the reference's primitive names; so a product meets the
LayerNorm in front of it and the activation behind it exactly as in a model written against
``folx_amd.numpy``.  The define-by-run front end stays the primary one; this is for models that exist as torch code."""

from __future__ import annotations

import logging
import operator

import numpy as np
import torch

from . import numpy as fnp
from .api import BatchedArray, FwdLaplArray
from .interpreter import ForwardLaplacianFn

aten = torch.ops.aten

# Named functions: the reference reaches its attention kernel through the NAME of a jitted function
# (``register_function('_multi_head_self_attention', ...)``, folx/experimental/pallas/attention/__init__.py:45, looked
# up by ``eval_pjit``, folx/interpreter.py:186-200).  The torch counterpart is a library operation: while a model is
# being traced the function below records ONE node, which the graph evaluation hands to the rule registered under the
# same key; outside a trace it is the plain differentiable arithmetic.
_LIB = torch.library.Library('folx_amd', 'DEF')
_LIB.define('multi_head_self_attention(Tensor q, Tensor k, Tensor v) -> Tensor')
_TRACING = [False]


def _mhsa_math(q, k, v):
    p = torch.softmax(torch.einsum('ihd,jhd->hij', q, k), dim=-1)
    return torch.einsum('hij,jhd->ihd', p, v)


_LIB.impl('multi_head_self_attention', _mhsa_math, 'CompositeExplicitAutograd')


def multi_head_self_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """``softmax(q k^T) v`` for per-sample tensors ``(n, heads, d)`` (no ``1 / sqrt(d)`` inside, as in the reference's
    ``folx.experimental.pallas.attention.multi_head_self_attention``): in a model traced by
    ``forward_laplacian_torch`` this is one equation and runs on the attention rule's kernel."""
    if _TRACING[0]:
        return torch.ops.folx_amd.multi_head_self_attention(q, k, v)
    return _mhsa_math(q, k, v)



def _is_t(v):
    from .wrapped_functions import Deferred

    return isinstance(v, (FwdLaplArray, BatchedArray, Deferred))


def _const(v):
    """Graph constants travel as numpy (float32 for floating point), python scalars as they are."""
    if isinstance(v, torch.Tensor):
        a = v.detach().cpu().numpy()
        return a.astype(np.float32) if np.issubdtype(a.dtype, np.floating) else a
    return v


def _shape(v):
    return tuple(fnp._shape(v)) if _is_t(v) else tuple(np.shape(v))


def _dims(d, nd):
    if d is None or (isinstance(d, (list, tuple)) and len(d) == 0):
        return tuple(range(nd))
    return tuple(int(i) % nd for i in (d if isinstance(d, (list, tuple)) else (d,)))


def _reduce(fn):
    def rule(a, dim=None, keepdim=False, dtype=None):
        nd = len(_shape(a))
        if nd == 0:
            return a
        return fn(a, axis=_dims(dim, nd), keepdims=bool(keepdim))

    return rule


def _view(a, shape):
    shape = [int(n) for n in shape]
    if -1 in shape:
        known = int(np.prod([n for n in shape if n != -1], dtype=int))
        shape[shape.index(-1)] = int(np.prod(_shape(a), dtype=int)) // max(known, 1)
    return fnp.reshape(a, tuple(shape))


def _expand(a, sizes, implicit=False):
    s = _shape(a)
    sizes = [int(n) for n in sizes]
    lead = len(sizes) - len(s)
    target = tuple(s[i - lead] if n == -1 else n for i, n in enumerate(sizes))
    if target == s:
        return a
    if len(target) == len(s):   # size-1 axes grow: a product with ones keeps it one rule (and sparse rows sparse)
        return fnp.multiply(a, np.ones(target, dtype=np.float32))
    return fnp.broadcast_to(a, target) if all(x == y for x, y in zip(target[lead:], s)) else \
        fnp.multiply(fnp.reshape(a, (1,) * lead + s), np.ones(target, dtype=np.float32))


def _slice(a, dim=0, start=None, end=None, step=1):
    nd = len(_shape(a))
    dim = dim % nd
    n = _shape(a)[dim]
    end = None if end is None or end >= n else end     # ATen passes sys.maxsize for "to the end"
    return fnp.getitem(a, (*([slice(None)] * dim), slice(start, end, step)))


def _select(a, dim, index):
    nd = len(_shape(a))
    return fnp.getitem(a, (*([slice(None)] * (dim % nd)), int(index)))


def _index(a, indices):
    if any(isinstance(i, BatchedArray) for i in indices):
        return _index_dynamic(a, list(indices))
    idx = tuple(slice(None) if i is None else np.asarray(i) for i in indices)
    return fnp.getitem(a, idx)


def _pow_scalar(a, e):
    if float(e) == int(e):
        return fnp.integer_pow(a, int(e))
    return fnp.power(a, float(e))


def _scaled(v, alpha):
    return v if alpha == 1 else fnp.multiply(v, float(alpha))


def _addmm(bias, a, b, beta=1, alpha=1):
    return fnp.add(_scaled(fnp.matmul(a, b), alpha), _scaled(bias, beta))


def _layer_norm(a, normalized_shape, weight, bias, eps):
    assert len(normalized_shape) == 1, 'native_layer_norm: only the last axis is normalised by the LayerNorm rule'
    return fnp.layer_norm(a, weight, bias, float(eps)), None, None


def _softplus(a, beta=1.0, threshold=20.0):
    if float(beta) == 1.0:
        return fnp.softplus(a)
    return fnp.multiply(fnp.softplus(fnp.multiply(a, float(beta))), 1.0 / float(beta))


def _squeeze(a, dims=None):
    s = _shape(a)
    ds = _dims(dims, len(s)) if dims is not None else tuple(range(len(s)))
    return fnp.reshape(a, tuple(n for i, n in enumerate(s) if not (i in ds and n == 1)))


def _max_dim(arg_fn, val_fn):
    def rule(a, dim, keepdim=False):
        v, i = val_fn(a, axis=int(dim)), arg_fn(a, axis=int(dim))
        if keepdim:
            v, i = fnp.expand_dims(v, int(dim)), np.expand_dims(np.asarray(i), int(dim)) if not _is_t(i) else i
        return v, i

    return rule


class _OnDemand:
    """An output of a multi-output operation that is only computed when the graph reads it."""

    def __init__(self, make):
        self.make = make


def _scan_with_indices(scan_fn, arg_fn):
    """``cummax`` / ``cummin``: values from the scan; indices (no derivatives) = the arg-extremum over each prefix,
    from an (n, n) masked copy, built only if the graph reads them."""
    def rule(a, dim):
        s = _shape(a)
        ax = int(dim) % len(s)
        n = s[ax]

        def indices():
            v = fnp.stop_gradient(a)
            big = np.float32(np.finfo(np.float32).max) * (1.0 if arg_fn is fnp.argmin else -1.0)
            keep = np.tril(np.ones((n, n), dtype=bool)).reshape((n,) + (1,) * (len(s) - 1 - ax) + (n,))
            rows = fnp.expand_dims(fnp.moveaxis(v, ax, -1), ax)            # (..., 1, ..., n): prefix i reads entries <= i
            full = fnp.where(keep, rows, big)
            return arg_fn(full, axis=-1)

        return scan_fn(a, axis=ax), _OnDemand(indices)

    return rule


def _item(a, i):
    v = a[i]
    return v.make() if isinstance(v, _OnDemand) else v


def _vector_norm(a, ord=2, dim=None, keepdim=False, dtype=None):
    nd = len(_shape(a))
    axes = _dims(dim, nd)
    o = float(ord)
    if o == 2.0:
        out = fnp.sqrt(fnp.sum(fnp.square(a), axis=axes, keepdims=bool(keepdim)))
    elif o == 1.0:
        out = fnp.sum(fnp.abs(a), axis=axes, keepdims=bool(keepdim))
    elif o == float('inf'):
        out = _fold_axes(fnp.amax, fnp.abs(a), axes, keepdim)
    elif o == -float('inf'):
        out = _fold_axes(fnp.amin, fnp.abs(a), axes, keepdim)
    else:
        out = fnp.power(fnp.sum(fnp.power(fnp.abs(a), o), axis=axes, keepdims=bool(keepdim)), 1.0 / o)
    return out


def _var(root):
    def rule(a, dim=None, correction=1, keepdim=False):
        nd = len(_shape(a))
        axes = _dims(dim, nd)
        n = int(np.prod([_shape(a)[i] for i in axes], dtype=int))
        c = 1 if correction is None else correction
        centred = fnp.subtract(a, fnp.mean(a, axis=axes, keepdims=True))
        v = fnp.multiply(fnp.sum(fnp.square(centred), axis=axes, keepdims=bool(keepdim)), 1.0 / max(n - float(c), 1e-30))
        return fnp.sqrt(v) if root else v

    return rule


def _split(a, size, dim=0):
    s = _shape(a)
    dim = int(dim) % len(s)
    sizes = [int(n) for n in size] if isinstance(size, (list, tuple)) else \
        [min(int(size), s[dim] - lo) for lo in range(0, s[dim], int(size))]
    out, lo = [], 0
    for n in sizes:
        out.append(_slice(a, dim, lo, lo + n))
        lo += n
    return tuple(out)


def _triangle(lower):
    def rule(a, diagonal=0):
        n, m = _shape(a)[-2:]
        keep = (np.tril if lower else np.triu)(np.ones((n, m), dtype=np.float32), int(diagonal))
        return fnp.multiply(a, keep)

    return rule


def _roll(a, shifts, dims=()):
    if not dims:   # the flattened array is rolled
        return fnp.reshape(fnp.roll(fnp.reshape(a, (-1,)), int(shifts[0]), 0), _shape(a))
    for sh, ax in zip(shifts, dims):
        a = fnp.roll(a, int(sh), int(ax) % len(_shape(a)))
    return a


def _masked_fill(a, mask, value):
    return fnp.where(mask, value if _is_t(value) else np.float32(value), a)


def _gather(a, dim, index, sparse_grad=False):
    """``out[i][j][k] = a[i][index[i][j][k]][k]`` (for dim 1): integer-array indexing with the other axes' own positions."""
    if isinstance(index, BatchedArray):
        assert tuple(index.shape) == tuple(n if ax != int(dim) % len(_shape(a)) else index.shape[ax] for ax, n in enumerate(_shape(a))), \
            'gather with walker-dependent indices: the index covers the other axes whole'
        return _select_along(a, index, int(dim))
    idx = np.asarray(index)
    nd = idx.ndim
    dim = int(dim) % nd
    grids = np.meshgrid(*[np.arange(n) for n in idx.shape], indexing='ij') if nd else []
    return fnp.getitem(a, tuple(idx if ax == dim else grids[ax] for ax in range(nd)))


def _sdpa(q, k, v, dropout_p=0.0, is_causal=False, attn_mask=None, scale=None, **_):
    """``softmax(q k^T scale (+ mask)) v`` with q, k, v ``(..., H, n, d)``: the attention rule when nothing is masked
    (one leading batch axis of extent one at most), the product and softmax rules otherwise."""
    assert float(dropout_p) == 0.0, 'scaled_dot_product_attention: dropout has no forward Laplacian'
    sq, sk = _shape(q), _shape(k)
    d, n, m = sq[-1], sq[-2], sk[-2]
    sc = float(scale) if scale is not None else 1.0 / float(np.sqrt(d))
    lead = sq[:-3]
    if attn_mask is None and not is_causal and n == m and all(x == 1 for x in lead) and len(sq) >= 3 and sq == sk == _shape(v):
        H = sq[-3]
        to_nhd = lambda t: fnp.transpose(fnp.reshape(t, (H, n, d)), (1, 0, 2))    # noqa: E731
        o = fnp.multi_head_self_attention(fnp.multiply(to_nhd(q), sc), to_nhd(k), to_nhd(v))
        return fnp.reshape(fnp.transpose(o, (1, 0, 2)), sq)
    scores = fnp.multiply(fnp.matmul(q, fnp.swapaxes(k, -1, -2)), sc)
    if is_causal:
        scores = fnp.where(np.tril(np.ones((n, m), dtype=bool)), scores, np.float32(-1e30))
    if attn_mask is not None:
        am = attn_mask
        if not _is_t(am) and np.asarray(am).dtype == bool:
            scores = fnp.where(np.asarray(am), scores, np.float32(-1e30))
        else:
            scores = fnp.add(scores, am)
    return fnp.matmul(fnp.softmax(scores, axis=-1), v)


def _cdist(a, b, p=2.0, compute_mode=None):
    diff = fnp.subtract(fnp.expand_dims(a, -2), fnp.expand_dims(b, -3))
    return _vector_norm(diff, p, (-1,), False)


def _log_sigmoid(a):
    out = fnp.negative(fnp.softplus(fnp.negative(a)))
    return out, None


def _elu(a, alpha=1.0, scale=1.0, input_scale=1.0):
    """``scale * (x > 0 ? x : alpha * (exp(input_scale * x) - 1))`` (selu and celu arrive in this form)."""
    if float(input_scale) == 1.0:
        out = fnp.elu(a, float(alpha))
    else:
        out = fnp.where(fnp.greater(fnp.stop_gradient(a), 0.0), a,
                        fnp.multiply(fnp.expm1(fnp.multiply(a, float(input_scale))), float(alpha)))
    return out if float(scale) == 1.0 else fnp.multiply(out, float(scale))


def _solve_ex(A, B, left=True, check_errors=False):
    if left:
        return fnp.solve(A, B), None, None, None
    # X A = B  <=>  A^T X^T = B^T
    vec = len(_shape(B)) == len(_shape(A)) - 1
    Bt = B if vec else fnp.swapaxes(B, -1, -2)
    X = fnp.solve(fnp.swapaxes(A, -1, -2), Bt)
    return (X if vec else fnp.swapaxes(X, -1, -2)), None, None, None


def _div_mode(a, b, rounding_mode=None):
    q = fnp.divide(a, b)
    if rounding_mode is None:
        return q
    return fnp.trunc(q) if rounding_mode == 'trunc' else fnp.floor(q)


def _prod_all(a, dtype=None):
    return fnp.prod(fnp.reshape(a, (-1,)), axis=0)


def _index_tuple(nd, dim, item):
    return (*([slice(None)] * (int(dim) % nd)), item)


def _copy(dst, src, non_blocking=False):
    """The functional form of ``dst.copy_(src)``: ``src`` with the shape of ``dst``."""
    return _expand(src, _shape(dst)) if _shape(src) != _shape(dst) else src


def _slice_scatter(a, src, dim=0, start=None, end=None, step=1):
    n = _shape(a)[int(dim) % len(_shape(a))]
    end = None if end is None or end >= n else end
    return fnp.scatter(a, _index_tuple(len(_shape(a)), dim, slice(start, end, step)), src, 'set')


def _select_scatter(a, src, dim, index):
    return fnp.scatter(a, _index_tuple(len(_shape(a)), dim, int(index)), src, 'set')


def _index_put(a, indices, values, accumulate=False):
    idx = tuple(slice(None) if i is None else np.asarray(i) for i in indices)
    return fnp.scatter(a, idx, values, 'add' if accumulate else 'set')


def _repeat(a, repeats):
    reps = [int(r) for r in repeats]
    s = _shape(a)
    if len(reps) > len(s):
        a = fnp.reshape(a, (1,) * (len(reps) - len(s)) + s)
    return fnp.tile(a, tuple(reps))


def _constant_pad(a, pad, value=0.0):
    nd = len(_shape(a))
    cfg = [(0, 0, 0)] * nd
    for i in range(len(pad) // 2):          # pairs run from the LAST axis backwards; negative widths crop
        cfg[nd - 1 - i] = (int(pad[2 * i]), int(pad[2 * i + 1]), 0)
    return fnp.lax_pad(a, np.float32(value), tuple(cfg))


def _extreme_all(fn):
    def rule(a):
        return fn(fnp.reshape(a, (-1,)), axis=0)

    return rule


def _frac(a):
    return fnp.subtract(a, fnp.trunc(a))


def _py_mod(a, b):
    """Python-style remainder ``a - b floor(a / b)`` (``torch.remainder``); the quotient is piecewise constant."""
    return fnp.subtract(a, fnp.multiply(b, fnp.floor(fnp.divide(fnp.stop_gradient(a), fnp.stop_gradient(b) if _is_t(b) else b))))


def _lerp(a, b, w):
    return fnp.add(a, fnp.multiply(w, fnp.subtract(b, a)))


def _xlogy(a, b):
    return fnp.multiply(a, fnp.log(b))


def _dist(a, b, p=2):
    return _vector_norm(fnp.subtract(a, b), p, None, False)


def _logcumsumexp(a, dim):
    """Shifted by the (derivative-free) maximum along the axis, like ``logsumexp``."""
    nd = len(_shape(a))
    ax = int(dim) % nd
    m = fnp.amax_const(a, (ax,), keepdims=True)
    return fnp.add(fnp.log(fnp.cumsum(fnp.exp(fnp.subtract(a, m)), axis=ax)), m)


def _loss(pointwise):
    def rule(a, b, reduction=1, *extra):
        v = pointwise(fnp.subtract(a, b), *extra)
        return v if reduction == 0 else (fnp.mean(v) if reduction == 1 else fnp.sum(v))

    return rule


def _huber(diff, delta=1.0):
    """``0.5 d^2`` for ``|d| < delta``, ``delta (|d| - 0.5 delta)`` beyond."""
    delta = float(delta)
    ad = fnp.abs(diff)
    return fnp.where(fnp.less(fnp.stop_gradient(ad), delta), fnp.multiply(fnp.square(diff), 0.5),
                     fnp.multiply(fnp.subtract(ad, 0.5 * delta), delta))


def _smooth_l1(diff, beta=1.0):
    beta = float(beta)
    return fnp.abs(diff) if beta == 0.0 else fnp.multiply(_huber(diff, beta), 1.0 / beta)


def _glu(a, dim=-1):
    s = _shape(a)
    ax = int(dim) % len(s)
    h = s[ax] // 2
    return fnp.multiply(_slice(a, ax, 0, h), fnp.sigmoid(_slice(a, ax, h, 2 * h)))


def _hard(lo, hi, scale, times_x):
    """``clip(x + 3, 0, 6) / 6`` family."""
    def rule(a):
        g = fnp.multiply(fnp.clip(fnp.add(a, 3.0), lo, hi), scale)
        return fnp.multiply(a, g) if times_x else g

    return rule


def _shrink(soft):
    def rule(a, lambd=0.5):
        lam = float(lambd)
        v = fnp.stop_gradient(a)
        if soft:
            return fnp.where(fnp.greater(v, lam), fnp.subtract(a, lam), fnp.where(fnp.less(v, -lam), fnp.add(a, lam), np.float32(0.0)))
        return fnp.where(fnp.logical_or(fnp.greater(v, lam), fnp.less(v, -lam)), a, np.float32(0.0))

    return rule


def _trilinear(i1, i2, i3, expand1, expand2, expand3, sumdim, unroll_dim=1):
    """``(i1.unsqueeze(expand1) * i2.unsqueeze(expand2) * i3.unsqueeze(expand3)).sum(sumdim)`` (what ``bilinear`` lowers to)."""
    def grow(t, dims):
        for dm in sorted(int(v) for v in dims):
            t = fnp.expand_dims(t, dm) if _is_t(t) else (t.unsqueeze(dm) if isinstance(t, torch.Tensor) else np.expand_dims(t, dm))
        return t

    prod = fnp.multiply(fnp.multiply(grow(i1, expand1), grow(i2, expand2)), grow(i3, expand3))
    return fnp.sum(prod, axis=tuple(int(v) for v in sumdim))


def _values_of(a):
    """The values of a triplet / walker-dependent array as a torch tensor (B, *shape), or None for a constant."""
    from .wrapped_functions import force

    a = force(a)
    if isinstance(a, FwdLaplArray):
        return a.x
    if isinstance(a, BatchedArray):
        return a.data
    return None


def _select_along(a, index: BatchedArray, axis: int):
    """``take_along_axis(a, index, axis)`` for indices that differ per walker (the positions of a sort, an arg-maximum):
    a 0 / 1 selection ``index == m`` over the ``n`` entries of the axis, multiplied in and summed -- linear in ``a``,
    ``n`` times the work of a static gather."""
    s = _shape(a)
    ax = axis % len(s)
    n = s[ax]
    pick = index.data.unsqueeze(ax + 2) == torch.arange(n, device=index.data.device).reshape((n,) + (1,) * (len(s) - 1 - ax))
    src = fnp.expand_dims(a, ax)                                       # (..., 1, n, ...): broadcast over the picked slot
    return fnp.sum(fnp.where(BatchedArray(pick), src, np.float32(0.0)), axis=ax + 1)


def _sort(a, dim=-1, descending=False, stable=False):
    v = _values_of(a)
    if v is None:
        r = torch.sort(torch.as_tensor(a), dim=int(dim), descending=bool(descending))
        return _const(r.values), _const(r.indices)
    ax = int(dim) % (v.dim() - 1)
    idx = BatchedArray(torch.argsort(v, dim=ax + 1, descending=bool(descending), stable=True))
    return (_select_along(a, idx, ax) if _is_t(a) and not isinstance(a, BatchedArray) else
            BatchedArray(torch.gather(v, ax + 1, idx.data))), idx


def _topk(a, k, dim=-1, largest=True, sorted=True):
    v = _values_of(a)
    if v is None:
        r = torch.topk(torch.as_tensor(a), int(k), dim=int(dim), largest=bool(largest))
        return _const(r.values), _const(r.indices)
    ax = int(dim) % (v.dim() - 1)
    idx = BatchedArray(torch.topk(v, int(k), dim=ax + 1, largest=bool(largest)).indices)
    return (_select_along(a, idx, ax) if not isinstance(a, BatchedArray) else BatchedArray(torch.gather(v, ax + 1, idx.data))), idx


def _index_dynamic(a, indices):
    """``a[i0, i1, ...]`` where some integer arrays differ per walker: the indexed axes (consecutive ones) are flattened
    into one, the flat position ``sum_j i_j stride_j`` is formed per walker, and the entries are picked by
    ``_select_along``."""
    s = _shape(a)
    where_ = [i for i, ix in enumerate(indices) if ix is not None]
    assert where_ == list(range(where_[0], where_[-1] + 1)), 'index arrays on consecutive axes only'
    lo, hi = where_[0], where_[-1] + 1
    dims = s[lo:hi]
    dev = next(ix.data.device for ix in indices if isinstance(ix, BatchedArray))
    B = next(ix.data.shape[0] for ix in indices if isinstance(ix, BatchedArray))
    flat, stride = 0, 1
    for ix, n in zip(reversed(indices[lo:hi]), reversed(dims)):
        t = ix.data.long() if isinstance(ix, BatchedArray) else torch.as_tensor(np.asarray(ix), device=dev).long()[None]
        flat = flat + torch.where(t < 0, t + n, t) * stride
        stride *= n
    ishape = tuple(flat.shape[1:])
    flat = flat.expand(B, *ishape)
    # (lead..., N, tail...) -> pick along N for every index entry
    src = fnp.reshape(a, (*s[:lo], int(np.prod(dims, dtype=int)), *s[hi:]))
    lead, tail = s[:lo], s[hi:]
    k = int(np.prod(ishape, dtype=int))
    idx = flat.reshape(B, *([1] * len(lead)), k, *([1] * len(tail))).expand(B, *lead, k, *tail)
    out = _select_along(src, BatchedArray(idx), lo)
    return fnp.reshape(out, (*lead, *ishape, *tail))


def _arg(fn, a, dim, keepdim):
    if dim is None:
        return fn(fnp.reshape(a, (-1,)), axis=0)
    out = fn(a, axis=int(dim))
    return fnp.expand_dims(out, int(dim)) if keepdim else out


def _group_norm(a, weight, bias, N, C, HxW, group, eps):
    """Normalisation over each group of ``C / group`` channels and all positions behind them; (out, mean, rstd)."""
    s = _shape(a)
    out = fnp.layer_norm(fnp.reshape(a, (int(N), int(group), -1)), None, None, float(eps))
    out = fnp.reshape(out, s)
    per_channel = (1, int(C)) + (1,) * (len(s) - 2)
    shaped = lambda t: fnp.reshape(t, per_channel) if _is_t(t) else t.reshape(per_channel)    # noqa: E731  (numpy or torch constant)
    if weight is not None:
        out = fnp.multiply(out, shaped(weight))
    if bias is not None:
        out = fnp.add(out, shaped(bias))
    return out, None, None


def _clamp(a, lo=None, hi=None):
    return fnp.clip(a, lo, hi)


def _identity(a, *_, **__):
    return a


# ATen operation -> the function of the same meaning (which finds its rule in the registry)
RULES = {
    aten.add.Tensor: lambda a, b, alpha=1: fnp.add(a, _scaled(b, alpha)),
    aten.add.Scalar: lambda a, b, alpha=1: fnp.add(a, float(b) * float(alpha)),
    aten.sub.Tensor: lambda a, b, alpha=1: fnp.subtract(a, _scaled(b, alpha)),
    aten.sub.Scalar: lambda a, b, alpha=1: fnp.subtract(a, float(b) * float(alpha)),
    aten.rsub.Scalar: lambda a, b, alpha=1: fnp.subtract(float(b), _scaled(a, alpha)),
    aten.mul.Tensor: fnp.multiply, aten.mul.Scalar: lambda a, b: fnp.multiply(a, float(b)),
    aten.div.Tensor: fnp.divide, aten.div.Scalar: lambda a, b: fnp.multiply(a, 1.0 / float(b)),
    aten.neg.default: fnp.negative, aten.reciprocal.default: fnp.reciprocal,
    aten.tanh.default: fnp.tanh, aten.sin.default: fnp.sin, aten.cos.default: fnp.cos, aten.exp.default: fnp.exp,
    aten.log.default: fnp.log, aten.sqrt.default: fnp.sqrt, aten.rsqrt.default: fnp.rsqrt,
    aten.sigmoid.default: fnp.sigmoid, aten.silu.default: fnp.silu, aten.relu.default: fnp.relu,
    aten.gelu.default: lambda a, approximate='none': fnp.gelu(a, approximate=(approximate == 'tanh')),
    aten.erf.default: fnp.erf, aten.erfc.default: fnp.erfc, aten.erfinv.default: fnp.erf_inv, aten.abs.default: fnp.abs,
    aten.expm1.default: fnp.expm1, aten.log1p.default: fnp.log1p, aten.sinh.default: fnp.sinh,
    aten.cosh.default: fnp.cosh, aten.tan.default: fnp.tan, aten.atan.default: fnp.arctan,
    aten.asin.default: fnp.arcsin, aten.acos.default: fnp.arccos, aten.asinh.default: fnp.arcsinh,
    aten.acosh.default: fnp.arccosh, aten.atanh.default: fnp.arctanh, aten.exp2.default: fnp.exp2,
    aten.lgamma.default: fnp.lgamma, aten.digamma.default: fnp.digamma, aten.atan2.default: fnp.arctan2,
    aten.softplus.default: _softplus, aten.elu.default: _elu,
    aten.leaky_relu.default: lambda a, negative_slope=0.01: fnp.leaky_relu(a, negative_slope),
    aten.pow.Tensor_Scalar: _pow_scalar, aten.pow.Tensor_Tensor: fnp.power, aten.pow.Scalar: lambda b, e: fnp.power(float(b), e),
    aten.square.default: fnp.square,
    aten.mm.default: fnp.matmul, aten.bmm.default: fnp.matmul, aten.matmul.default: fnp.matmul, aten.addmm.default: _addmm,
    aten.dot.default: fnp.vdot, aten.mv.default: fnp.matmul,
    aten.t.default: lambda a: a if len(_shape(a)) < 2 else fnp.swapaxes(a, -1, -2),
    aten.transpose.int: lambda a, d0, d1: fnp.swapaxes(a, int(d0), int(d1)),
    aten.permute.default: lambda a, dims: fnp.transpose(a, [int(d) for d in dims]),
    aten.view.default: _view, aten.reshape.default: _view, aten._unsafe_view.default: _view,
    aten.expand.default: _expand,
    aten.unsqueeze.default: lambda a, dim: fnp.expand_dims(a, int(dim)),
    aten.squeeze.dim: lambda a, dim: _squeeze(a, (dim,)), aten.squeeze.dims: _squeeze, aten.squeeze.default: _squeeze,
    aten.slice.Tensor: _slice, aten.select.int: _select, aten.index.Tensor: _index,
    aten.cat.default: lambda ts, dim=0: fnp.concatenate(list(ts), axis=int(dim)),
    aten.stack.default: lambda ts, dim=0: fnp.stack(list(ts), axis=int(dim)),
    aten.flip.default: lambda a, dims: fnp.flip(a, tuple(int(d) for d in dims)) if len(dims) > 1 else fnp.flip(a, int(dims[0])),
    aten.sum.default: _reduce(fnp.sum), aten.sum.dim_IntList: _reduce(fnp.sum),
    aten.mean.default: _reduce(fnp.mean), aten.mean.dim: _reduce(fnp.mean),
    aten.amax.default: lambda a, dim=(), keepdim=False: _fold_axes(fnp.amax, a, dim, keepdim),
    aten.amin.default: lambda a, dim=(), keepdim=False: _fold_axes(fnp.amin, a, dim, keepdim),
    aten.max.dim: _max_dim(fnp.argmax, fnp.amax), aten.min.dim: _max_dim(fnp.argmin, fnp.amin),
    aten.prod.dim_int: lambda a, dim, keepdim=False, dtype=None: _fold_axes(fnp.prod, a, (dim,), keepdim),
    aten.cumsum.default: lambda a, dim, dtype=None: fnp.cumsum(a, axis=int(dim)),
    aten.cumprod.default: lambda a, dim, dtype=None: fnp.cumprod(a, axis=int(dim)),
    aten.cummax.default: _scan_with_indices(fnp.cummax, fnp.argmax), aten.cummin.default: _scan_with_indices(fnp.cummin, fnp.argmin),
    aten.unbind.int: lambda a, dim=0: tuple(_select(a, dim, i) for i in range(_shape(a)[int(dim) % len(_shape(a))])),
    aten._softmax.default: lambda a, dim, half=False: fnp.softmax(a, axis=int(dim)),
    aten._log_softmax.default: lambda a, dim, half=False: fnp.log_softmax(a, axis=int(dim)),
    aten.logsumexp.default: lambda a, dim, keepdim=False: _logsumexp(a, dim, keepdim),
    aten.native_layer_norm.default: _layer_norm,
    aten.where.self: fnp.where,
    aten.gt.Scalar: fnp.greater, aten.gt.Tensor: fnp.greater, aten.ge.Scalar: fnp.greater_equal, aten.ge.Tensor: fnp.greater_equal,
    aten.lt.Scalar: fnp.less, aten.lt.Tensor: fnp.less, aten.le.Scalar: fnp.less_equal, aten.le.Tensor: fnp.less_equal,
    aten.eq.Scalar: fnp.equal, aten.eq.Tensor: fnp.equal, aten.ne.Scalar: fnp.not_equal, aten.ne.Tensor: fnp.not_equal,
    aten.logical_and.default: fnp.logical_and, aten.logical_or.default: fnp.logical_or, aten.logical_not.default: fnp.logical_not,
    aten.clamp.default: _clamp, aten.clamp_min.default: lambda a, lo: fnp.clip(a, lo, None),
    aten.clamp_max.default: lambda a, hi: fnp.clip(a, None, hi),
    aten.minimum.default: fnp.minimum, aten.maximum.default: fnp.maximum,
    aten.clone.default: _identity, aten.alias.default: _identity, aten.contiguous.default: _identity,
    aten._to_copy.default: _identity, aten.lift_fresh_copy.default: _identity,
    aten.detach.default: fnp.stop_gradient,
    aten._linalg_slogdet.default: lambda A: (*fnp.slogdet(A), None, None),
    aten._linalg_det.default: lambda A: (fnp.det(A), None, None),
    aten.linalg_inv_ex.default: lambda A, check_errors=False: (fnp.inv(A), None),
    aten._linalg_solve_ex.default: _solve_ex,
    operator.getitem: _item,
    aten.sign.default: fnp.sign, aten.sgn.default: fnp.sign,
    # a constant that only borrows the SHAPE of a data tensor (the seed of a gradient taken inside the function, ...)
    aten.ones_like.default: lambda a, **_: np.ones(_shape(a), np.float32),
    aten.zeros_like.default: lambda a, **_: np.zeros(_shape(a), np.float32),
    aten.full_like.default: lambda a, value, **_: np.full(_shape(a), float(value), np.float32),
    aten.new_ones.default: lambda a, size, **_: np.ones(tuple(int(n) for n in size), np.float32),
    aten.new_zeros.default: lambda a, size, **_: np.zeros(tuple(int(n) for n in size), np.float32),
    aten.new_full.default: lambda a, size, value, **_: np.full(tuple(int(n) for n in size), float(value), np.float32),
    aten.index_select.default: lambda a, dim, index: fnp.take(a, np.asarray(index), axis=int(dim)),
    aten.take.default: lambda a, index: fnp.take(a, np.asarray(index)),
    aten.squeeze_.dim: lambda a, dim: _squeeze(a, (dim,)), aten.unsqueeze_.default: lambda a, dim: fnp.expand_dims(a, int(dim)),
    aten._safe_softmax.default: lambda a, dim, dtype=None: fnp.softmax(a, axis=int(dim)),
    aten.linalg_vector_norm.default: _vector_norm,
    aten.var.correction: _var(False), aten.std.correction: _var(True),
    aten.split.Tensor: _split, aten.split_with_sizes.default: _split,
    aten.tril.default: _triangle(True), aten.triu.default: _triangle(False),
    aten.diagonal.default: lambda a, offset=0, dim1=0, dim2=1: fnp.diagonal(fnp.moveaxis(a, (int(dim1), int(dim2)), (-2, -1)), int(offset)),
    aten.trace.default: fnp.trace,
    aten.baddbmm.default: _addmm, aten.addmv.default: _addmm, aten.addbmm.default:
        lambda bias, a, b, beta=1, alpha=1: fnp.add(_scaled(fnp.sum(fnp.matmul(a, b), axis=0), alpha), _scaled(bias, beta)),
    aten.addcmul.default: lambda a, t1, t2, value=1: fnp.add(a, _scaled(fnp.multiply(t1, t2), value)),
    aten.addcdiv.default: lambda a, t1, t2, value=1: fnp.add(a, _scaled(fnp.divide(t1, t2), value)),
    aten.masked_fill.Scalar: _masked_fill, aten.masked_fill.Tensor: _masked_fill,
    aten.roll.default: _roll,
    aten.gather.default: _gather,
    aten._linalg_check_errors.default: lambda *a, **k: None,
    aten.mish.default: lambda a: fnp.multiply(a, fnp.tanh(fnp.softplus(a))),
    aten.sort.default: _sort, aten.sort.stable: lambda a, stable=False, dim=-1, descending=False: _sort(a, dim, descending),
    aten.topk.default: _topk,
    aten.norm.ScalarOpt_dim: lambda a, p=2, dim=None, keepdim=False: _vector_norm(a, 2 if p is None else p, dim, keepdim),
    aten.norm.Scalar: lambda a, p=2: _vector_norm(a, p, None, False),
    aten.native_group_norm.default: _group_norm,
    aten.argmax.default: lambda a, dim=None, keepdim=False: _arg(fnp.argmax, a, dim, keepdim),
    aten.argmin.default: lambda a, dim=None, keepdim=False: _arg(fnp.argmin, a, dim, keepdim),
    aten.empty_like.default: lambda a, **_: np.zeros(_shape(a), np.float32),
    aten.copy.default: _copy, aten.slice_scatter.default: _slice_scatter, aten.select_scatter.default: _select_scatter,
    aten.index_put.default: _index_put,
    aten.repeat.default: _repeat, aten.constant_pad_nd.default: _constant_pad,
    aten.max.default: _extreme_all(fnp.amax), aten.min.default: _extreme_all(fnp.amin),
    aten.floor.default: fnp.floor, aten.ceil.default: fnp.ceil, aten.round.default: fnp.round, aten.trunc.default: fnp.trunc,
    aten.frac.default: _frac, aten.fmod.Scalar: fnp.remainder, aten.fmod.Tensor: fnp.remainder,
    aten.remainder.Scalar: _py_mod, aten.remainder.Tensor: _py_mod,
    aten.lerp.Scalar: _lerp, aten.lerp.Tensor: _lerp,
    aten.hypot.default: lambda a, b: fnp.sqrt(fnp.add(fnp.square(a), fnp.square(b))),
    aten.logaddexp.default: fnp.logaddexp, aten.xlogy.Tensor: _xlogy, aten.dist.default: _dist,
    aten.logcumsumexp.default: _logcumsumexp,
    aten.mse_loss.default: _loss(fnp.square), aten.l1_loss.default: _loss(fnp.abs),
    aten.huber_loss.default: _loss(_huber), aten.smooth_l1_loss.default: _loss(_smooth_l1),
    aten.glu.default: _glu,
    aten.hardswish.default: _hard(0.0, 6.0, 1.0 / 6.0, True), aten.hardsigmoid.default: _hard(0.0, 6.0, 1.0 / 6.0, False),
    aten.relu6.default: lambda a: fnp.clip(a, 0.0, 6.0),
    aten.softshrink.default: _shrink(True), aten.hardshrink.default: _shrink(False),
    aten.threshold.default: lambda a, threshold, value: fnp.where(fnp.greater(fnp.stop_gradient(a), float(threshold)), a, np.float32(value)),
    aten.rrelu_with_noise.default: lambda a, noise, lower=0.125, upper=1.0 / 3.0, training=False, generator=None:
        fnp.leaky_relu(a, (float(lower) + float(upper)) / 2.0),
    aten._prelu_kernel.default: lambda a, w: fnp.where(fnp.greater(fnp.stop_gradient(a), 0.0), a, fnp.multiply(a, w)),
    aten._trilinear.default: _trilinear,
    aten.unsafe_split.Tensor: _split, aten.unsafe_split_with_sizes.default: _split, aten.unsafe_chunk.default:
        lambda a, chunks, dim=0: _split(a, -(-_shape(a)[int(dim) % len(_shape(a))] // int(chunks)), dim),
    aten.celu.default: lambda a, alpha=1.0: _elu(a, float(alpha), 1.0, 1.0 / float(alpha)),
    aten.clamp.Tensor: _clamp, aten.clamp_min.Tensor: lambda a, lo: fnp.maximum(a, lo), aten.clamp_max.Tensor: lambda a, hi: fnp.minimum(a, hi),
    aten.div.Tensor_mode: _div_mode, aten.div.Scalar_mode: _div_mode,
    aten.prod.default: _prod_all,
    aten.where.ScalarSelf: fnp.where, aten.where.ScalarOther: fnp.where, aten.where.Scalar: fnp.where,
    aten.log_sigmoid_forward.default: _log_sigmoid,
    aten.hardtanh.default: lambda a, lo=-1.0, hi=1.0: fnp.clip(a, float(lo), float(hi)),
    aten._scaled_dot_product_flash_attention_for_cpu.default: lambda q, k, v, dropout_p=0.0, is_causal=False, attn_mask=None,
        scale=None: (_sdpa(q, k, v, dropout_p, is_causal, attn_mask, scale), None),
    aten._scaled_dot_product_attention_math.default: lambda q, k, v, attn_mask=None, dropout_p=0.0, is_causal=False,
        dropout_mask=None, scale=None, enable_gqa=False: (_sdpa(q, k, v, dropout_p, is_causal, attn_mask, scale), None),
    aten._cdist_forward.default: _cdist,
    torch.ops.folx_amd.multi_head_self_attention.default: fnp.multi_head_self_attention,
}


def _amax_values(a, dims=(), keepdim=False):
    s = _shape(a)
    axes = _dims(dims, len(s))
    return fnp.amax_const(a, axes, keepdims=bool(keepdim))


def _fold_axes(fn, a, dims, keepdim):
    s = _shape(a)
    axes = sorted(_dims(dims, len(s)), reverse=True)
    out = a
    for ax in axes:
        out = fn(out, axis=ax)
    if keepdim:
        out = fnp.reshape(out, tuple(1 if i in axes else n for i, n in enumerate(s)))
    return out


def _logsumexp(a, dims, keepdim):
    s = _shape(a)
    axes = _dims(dims, len(s))
    assert len(axes) == 1, 'logsumexp: one axis'
    out = fnp.logsumexp(a, axis=axes[0])[0]
    return fnp.expand_dims(out, axes[0]) if keepdim else out


def _functional_form(target):
    """``aten.add_.Tensor`` -> ``aten.add.Tensor`` when that has a rule, else None."""
    name = getattr(target, '_schema', None)
    if name is None:
        return None
    base = target._schema.name.split('::')[-1]
    if not base.endswith('_') or base.endswith('__'):
        return None
    packet = getattr(aten, base[:-1], None)
    functional = getattr(packet, target._overloadname, None) if packet is not None else None
    return functional if functional in RULES else None


def _disjoint_part_of_a_dead_tensor(part, at, order):
    """``part`` is one piece of a split / chunk / unbind whose source nobody reads any more (only the split itself
    does): updating the piece in place touches nothing else that the graph still looks at (the gates of a GRU cell)."""
    if part.target is not operator.getitem:
        return False
    split = part.args[0]
    if not isinstance(split, torch.fx.Node) or split.target not in _SPLITS:
        return False
    source = split.args[0]
    return isinstance(source, torch.fx.Node) and all(u is split or order[u] < order[at] for u in source.users)


_SPLITS = {aten.split.Tensor, aten.split_with_sizes.default, aten.unbind.int, aten.unsafe_split.Tensor,
           aten.unsafe_split_with_sizes.default, aten.unsafe_chunk.default}
_VIEWS = {aten.slice.Tensor, aten.select.int, aten.view.default, aten._unsafe_view.default, aten.reshape.default,
          aten.transpose.int, aten.permute.default, aten.t.default, aten.expand.default, aten.unsqueeze.default,
          aten.squeeze.dim, aten.squeeze.dims, aten.squeeze.default, aten.diagonal.default, aten.alias.default,
          aten.detach.default, aten.unbind.int, aten.split.Tensor, aten.split_with_sizes.default, operator.getitem}


def _generic(target):
    """An ATen operation without an entry above: the generic rule built from the operation itself, with the warning
    the reference gives for a primitive outside its registry (folx/wrapped_functions.py:609-614)."""
    def rule(*args, **kwargs):
        logging.warning(f'{target} has no forward-Laplacian rule; the following call computes the full Hessian of the operation')
        if any(isinstance(v, (list, tuple)) and _any_triplet(v) for v in args):
            # a list of tensors (block_diag, ...): the wrapped function takes its entries one by one
            spans, flat = [], []
            for v in args:
                if isinstance(v, (list, tuple)) and _any_triplet(v):
                    spans.append((len(flat), len(v)))
                    flat.extend(v)
                else:
                    spans.append(None)
                    flat.append(v)

            def packed(*a):
                it, full = 0, []
                for sp in spans:
                    if sp is None:
                        full.append(a[it])
                        it += 1
                    else:
                        full.append(list(a[it:it + sp[1]]))
                        it += sp[1]
                return target(*full, **kwargs)

            return fnp.call(packed, *flat)
        return fnp.call(lambda *a: target(*a, **kwargs), *args)

    return rule


def _tree(v, fn):
    if isinstance(v, (list, tuple)):
        return type(v)(_tree(t, fn) for t in v)
    if isinstance(v, dict):
        return {k: _tree(t, fn) for k, t in v.items()}
    return fn(v)


def _any_triplet(v):
    if isinstance(v, (list, tuple)):
        return any(_any_triplet(t) for t in v)
    if isinstance(v, dict):
        return any(_any_triplet(t) for t in v.values())
    return _is_t(v)


def fold_constants(gm: torch.fx.GraphModule):
    """Every equation whose inputs are all constants, evaluated once by torch itself on the host (the reference binds
    such equations eagerly while it interprets, folx/interpreter.py:222-245): node -> numpy array / scalar / tuple."""
    env = {}
    look = lambda a: env[a] if isinstance(a, torch.fx.Node) else a
    is_const = lambda a: not isinstance(a, torch.fx.Node) or a in env

    def all_const(v):
        if isinstance(v, (list, tuple)):
            return all(all_const(t) for t in v)
        if isinstance(v, dict):
            return all(all_const(t) for t in v.values())
        return is_const(v)

    for node in gm.graph.nodes:
        if node.op == 'get_attr':
            obj = gm
            for part in node.target.split('.'):
                obj = getattr(obj, part)
            env[node] = obj.detach() if isinstance(obj, torch.Tensor) else obj
        elif node.op == 'call_function' and all_const(node.args) and all_const(node.kwargs):
            args = torch.fx.node.map_arg(node.args, look)
            kwargs = torch.fx.node.map_arg(node.kwargs, look)
            with torch.no_grad():
                env[node] = node.target(*args, **kwargs)
    return {n: _tree(v, _const) for n, v in env.items()}


_WEIGHT_READERS = {aten.mm.default, aten.addmm.default, aten.bmm.default, aten.matmul.default, aten.mv.default,
                   aten.native_layer_norm.default}
_DEVICE_CONST_MIN = 256   # constants of at least this many floats live on the device between evaluations


def evaluate_graph(gm: torch.fx.GraphModule, inputs, consts=None):
    """One pass over the equations of a traced graph (folx/interpreter.py:218-264): constant equations come from
    ``fold_constants``, the others go through ``RULES``."""
    env = dict(fold_constants(gm) if consts is None else consts)
    it = iter(inputs)
    look = lambda a: env[a] if isinstance(a, torch.fx.Node) else a
    order = {n: i for i, n in enumerate(gm.graph.nodes)}
    for node in gm.graph.nodes:
        if node in env:
            continue
        if node.op == 'placeholder':
            env[node] = next(it)
        elif node.op == 'call_function':
            args = torch.fx.node.map_arg(node.args, look)
            kwargs = torch.fx.node.map_arg(node.kwargs, look)
            kwargs = {k: v for k, v in kwargs.items() if k not in ('dtype', 'device', 'layout', 'pin_memory', 'memory_format')}
            rule = RULES.get(node.target)
            functional = _functional_form(node.target) if rule is None else None
            if functional is not None:
                # an in-place update of an intermediate (inside a library function: ``tmp.add_(eps)``): the functional
                # operation, and the updated tensor is what its name means from here on.  Updates through views of the
                # caller's own tensors never get here (the trace is functionalized); a view updated in place would
                # leave its base behind, so that case raises.
                target_node = node.args[0]
                if not isinstance(target_node, torch.fx.Node) or target_node.op == 'placeholder' or \
                        (target_node.target in _VIEWS and not _disjoint_part_of_a_dead_tensor(target_node, node, order)):
                    raise NotImplementedError(f'{node.format_node()}: in-place update of an input or of a view')
                for view in target_node.users:   # a view taken BEFORE the update and read AFTER it would miss the update
                    if view.target in _VIEWS and order[view] < order[node] and any(order[w] > order[node] for w in view.users):
                        raise NotImplementedError(f'{node.format_node()}: in-place update of a tensor whose earlier '
                                                  f'view {view.name} is read afterwards')
                env[node] = env[target_node] = RULES[functional](*args, **kwargs)
                continue
            rule = rule or _generic(node.target)
            if node.target is aten.amax.default and node.users and all(u.target is aten.detach.default for u in node.users):
                rule = _amax_values   # max(...).detach(): the shift of a softmax / logsumexp carries no derivatives
            try:
                env[node] = rule(*args, **kwargs)
            except Exception:
                logging.error(f'forward Laplacian of {node.format_node()} failed')   # folx/interpreter.py:254-257
                raise
        elif node.op == 'output':
            return torch.fx.node.map_arg(node.args[0], look)
        else:
            raise NotImplementedError(f'graph node {node.op}')
    raise RuntimeError('graph without an output')


_NAMED = {}


def named_function(name: str, fn):
    """A torch function that the trace keeps as ONE equation, evaluated by the rule registered under ``name`` -- the
    reference looks jitted functions up by name the same way (``eval_pjit``, folx/interpreter.py:186-200:
    ``register_function('my_layer', rule)`` + ``jax.jit(my_layer)``).  Returns the function to call in the model: while
    ``forward_laplacian_torch`` traces, the call is a library operation ``folx_amd::<name>`` over its tensor arguments;
    otherwise it is ``fn`` itself.  Without a rule under ``name`` at evaluation time the function gets the generic
    rule (``wrap_forward_laplacian(fn)``).  ``fn`` takes tensors and returns a tensor or a tuple of tensors."""
    assert name.isidentifier(), 'the name becomes an operator name'
    if name in _NAMED:
        assert _NAMED[name][0] is fn, f'{name} already names another function'
        return _NAMED[name][1]

    single = [True]

    def impl(inputs):
        out = fn(*inputs)
        single[0] = not isinstance(out, (tuple, list))     # known once the operation has run (it runs while tracing)
        return [out] if single[0] else list(out)

    _LIB.define(f'{name}(Tensor[] inputs) -> Tensor[]')
    _LIB.impl(name, impl, 'CompositeExplicitAutograd')
    op = getattr(torch.ops.folx_amd, name).default

    def rule(inputs):
        from .wrapped_functions import get_laplacian, is_registered
        from .wrapper import wrap_forward_laplacian

        r = get_laplacian(name) if is_registered(name) else wrap_forward_laplacian(fn, name=name)
        out = r(tuple(inputs), {}, fnp.current_threshold())
        return list(out) if isinstance(out, (tuple, list)) else [out]

    RULES[op] = rule

    def call(*tensors):
        if not _TRACING[0]:
            return fn(*tensors)
        out = op(list(tensors))
        return out[0] if single[0] else tuple(out)

    call.__name__ = name
    _NAMED[name] = (fn, call)
    return call


class TracedForwardLaplacian(ForwardLaplacianFn):
    """``forward_laplacian_torch(fn, thr)``: ``f(x)`` takes one sample, ``f.batched(x)`` walkers, as for
    ``forward_laplacian``; the torch function is traced once per combination of input shapes, its constant
    equations are evaluated then, and the larger constants (weights) are uploaded once per device."""

    def __init__(self, fn, sparsity_threshold):
        self.torch_fn = fn
        self.graphs = {}
        self.constants = {}
        super().__init__(self._run, sparsity_threshold)

    def _graph(self, shapes):
        gm = self.graphs.get(shapes)
        if gm is None:
            from torch.fx.experimental.proxy_tensor import make_fx

            with torch.no_grad():
                examples = [torch.zeros(s, dtype=torch.float32) + 0.5 for s in shapes]
                _TRACING[0] = True
                try:
                    # in-place updates and slice assignments of the function become their functional forms
                    # (add_, copy_ into a view, index_put_ ... -> add, slice_scatter, index_put ...)
                    gm = self.graphs[shapes] = make_fx(torch.func.functionalize(self.torch_fn))(*examples)
                finally:
                    _TRACING[0] = False
            self.constants[shapes] = fold_constants(gm)
        return gm

    def _constants(self, shapes, device):
        key = (shapes, str(device))
        hit = self.constants.get(key)
        if hit is None:
            def place(v):
                if (isinstance(v, np.ndarray) and v.dtype == np.float32 and v.size >= _DEVICE_CONST_MIN
                        and device.type != 'cpu'):
                    return torch.as_tensor(np.ascontiguousarray(v)).to(device)
                return v
            # only what the product rules read (weights): they take device tensors as they are, and every other
            # rule keeps seeing host arrays, whatever the size of its constants
            hit = self.constants[key] = {n: (_tree(v, place) if n.users and all(u.target in _WEIGHT_READERS for u in n.users) else v)
                                         for n, v in self.constants[shapes].items()}
        return hit

    def _run(self, *lapl_args):
        shapes = tuple(tuple(a.shape) for a in lapl_args)
        gm = self._graph(shapes)
        return evaluate_graph(gm, lapl_args, self._constants(shapes, lapl_args[0].x.device))

    def invalidate(self):
        """Forget the traces (and the constants folded from them): the next call traces again, e.g. after the
        parameters of a traced module have changed."""
        self.graphs.clear()
        self.constants.clear()


def forward_laplacian_torch(fn, sparsity_threshold: int | float = 0) -> TracedForwardLaplacian:
    """The traced counterpart of ``forward_laplacian`` for a function (or ``torch.nn.Module``) written with torch:
    ``fn(*tensors)`` maps ONE sample to a tensor or a tuple / list / dict of tensors; every tensor argument is
    differentiated (one index space, in argument order)."""
    return TracedForwardLaplacian(fn, sparsity_threshold)

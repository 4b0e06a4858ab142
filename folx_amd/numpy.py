"""``jax.numpy``-shaped front end: the functions a model calls, each dispatched through the
rule registry under the primitive name the reference uses.

The reference traces ``jnp`` code into a jaxpr and interprets it (folx/interpreter.py:
127-264); here the same dispatch happens define-by-run: every function below looks up
``get_laplacian(<primitive>)`` and calls the rule with ``(args, kwargs,
sparsity_threshold)``.  Shapes and axes are per walker, as inside ``jax.vmap``.
"""

from __future__ import annotations

import contextlib
import threading

import numpy as np

from .api import BatchedArray, FwdLaplArray
from .wrapped_functions import get_laplacian, register_function

_state = threading.local()


def current_threshold() -> int:
    return getattr(_state, 'threshold', 0)


@contextlib.contextmanager
def sparsity_threshold(value: int):
    old = current_threshold()
    _state.threshold = int(value)
    try:
        yield
    finally:
        _state.threshold = old


def _call(name, args, kwargs=None):
    """Look the rule up and call it.  Deferred values among the arguments are evaluated first
    (also one level inside tuples and among the keyword values): only the functions below that
    know how to absorb one hand it on, through ``_call_keep``."""
    from .wrapped_functions import force

    kwargs = {k: force(v) for k, v in (kwargs or {}).items()}
    return get_laplacian(name, wrap_if_missing=True)(tuple(force(a) for a in args), kwargs, current_threshold())


def call(name_or_fn, *args, **kwargs):
    """Apply the rule registered under ``name_or_fn`` to ``args`` -- what the reference's interpreter
    does when it meets a primitive or a jitted function of that name (folx/interpreter.py:186-216).
    A callable that has no rule of its own (a torch function of per-walker tensors) goes through
    the generic rule (``folx_amd.wrapper.wrap_forward_laplacian``)."""
    return _call(name_or_fn, args, kwargs)


def _call_keep(name, args, kwargs=None):
    return get_laplacian(name, wrap_if_missing=True)(tuple(args), kwargs or {}, current_threshold())


def _is_triplet(a):
    from .wrapped_functions import Deferred

    return isinstance(a, (FwdLaplArray, Deferred))


def _shape(a):
    if isinstance(a, BatchedArray) or _is_triplet(a):
        return tuple(a.shape)
    return tuple(np.shape(a))


# elementwise -------------------------------------------------------------------------------
def _u(name):
    def fn(a):
        from .kernels import FUSED_ACTS
        from .wrapped_functions import LazyDot

        if isinstance(a, LazyDot) and name in FUSED_ACTS and a.kwargs.get('act') is None:
            return a.with_(act=name)  # Dense + activation: one rule where the kernels take the shape
        return _call(name, (a,))

    fn.__name__ = name
    return fn


tanh, exp, log, sqrt, rsqrt, square = _u('tanh'), _u('exp'), _u('log'), _u('sqrt'), _u('rsqrt'), _u('square')
sin, cos, abs, log1p, expm1 = _u('sin'), _u('cos'), _u('abs'), _u('log1p'), _u('expm1')
silu, softplus, sigmoid, logistic = _u('silu'), _u('softplus'), _u('sigmoid'), _u('logistic')
sinh, cosh, tan = _u('sinh'), _u('cosh'), _u('tan')
arcsin, arccos, arctan = _u('asin'), _u('acos'), _u('atan')
arcsinh, arccosh, arctanh = _u('asinh'), _u('acosh'), _u('atanh')
erf, erfc, erf_inv, cbrt = _u('erf'), _u('erfc'), _u('erf_inv'), _u('cbrt')
lgamma, digamma = _u('lgamma'), _u('digamma')
reciprocal, negative, sign, stop_gradient = _u('reciprocal'), _u('neg'), _u('sign'), _u('stop_gradient')


def integer_pow(a, n: int):
    return _call('integer_pow', (a,), {'y': int(n)})


def power(a, c):
    """``a ** c`` for ``a > 0``: a constant real exponent runs the fused scalar rule; an
    exponent that carries derivatives (or a constant base) goes through ``exp(c log a)``."""
    from .api import FwdLaplArray as _F

    if isinstance(c, _F) or not np.isscalar(c):
        if not isinstance(a, _F):
            return exp(multiply(c, np.log(np.asarray(a, dtype=np.float32))))
        return exp(multiply(c, log(a)))
    return _call('pow', (a,), {'y': float(c)})


def add(a, b):
    from .wrapped_functions import LazyDot, force

    for d, o in ((b, a), (a, b)):
        if not isinstance(d, LazyDot) or d._value is not None:  # an evaluated product is an ordinary triplet
            continue
        if not _is_triplet(o) and not isinstance(o, BatchedArray):
            # a constant vector along the feature axis in front of the activation: the bias
            if (d.kwargs.get('act') is None and d.kwargs.get('bias') is None and np.ndim(o) == 1
                    and _shape(o) == (d.shape[-1],)):
                return d.with_(bias=o)
        elif _is_triplet(o) and tuple(o.shape) == tuple(d.shape):
            return d.value_with_residual(force(o))  # skip connection: added in the product's epilogue
        break
    return _call('add', (a, b))


def subtract(a, b):
    return _call('sub', (a, b))


def multiply(a, b):
    from .wrapped_functions import LazyMul, force

    if _is_triplet(a) and _is_triplet(b) and tuple(a.shape) == tuple(b.shape) and len(a.shape) >= 2:
        return LazyMul(force(a), force(b), current_threshold())  # slogdet can take the factor on load
    return _call('mul', (a, b))


def divide(a, b):
    return _call('div', (a, b))


# linear algebra ----------------------------------------------------------------------------
def dot(h, W, b=None, residual=None, row_slice=None, act=None, norm=None):
    """``h @ W``: last axis of ``h`` against the first axis of the constant ``W``.

    Written plainly, ``tanh(dot(layer_norm(h, g, be), W) + bias) + skip`` runs as ONE rule where
    the kernels take the shape: ``dot`` absorbs a ``layer_norm``, a ``concatenate`` along the
    feature axis or a slice of rows in front of it, and returns a deferred value that absorbs the
    bias, the activation and the skip connection that follow (``wrapped_functions.Deferred``).

    The keyword form states the same fusion explicitly and evaluates at once: ``b`` bias,
    ``residual`` a triplet of the output shape, ``row_slice = (lo, hi)`` for
    ``h[..., lo:hi, :] @ W``, ``act`` a scalar function applied to ``h @ W + b`` (the residual is
    added to the activated result), ``norm = (gamma, beta, eps)`` a LayerNorm of ``h``."""
    from .wrapped_functions import LazyConcat, LazyDot, LazyLayerNorm, LazySlice, force

    if isinstance(h, LazyLayerNorm):
        assert norm is None, 'dot: the operand already is a layer_norm'
        h, norm = h.h, h
    elif isinstance(h, LazySlice) and row_slice is None and h.ndim >= 2 and h.axis == h.ndim - 2:
        h, row_slice = h.a, (h.lo, h.hi)
    elif not isinstance(h, LazyConcat):
        h = force(h)
    kwargs = {'bias': b, 'row_slice': row_slice, 'act': act, 'norm': norm}
    explicit = residual is not None or act is not None
    if explicit or not _is_triplet(h) or _is_triplet(W) or np.ndim(W) != 2:
        return _call_keep('dot_general', (h, force(W)), {**kwargs, 'residual': force(residual)})
    lead = tuple(h.shape[:-1])
    if row_slice is not None:
        lead = (*lead[:-1], row_slice[1] - row_slice[0])
    return LazyDot(h, W, kwargs, (*lead, int(np.shape(W)[1])), current_threshold())


def layer_norm(h, gamma=None, beta=None, eps=1e-5, lazy=True):
    """LayerNorm over the last axis (one fused rule; same result as the primitive chain).  The
    result is deferred: products that can take LayerNorm into their own rule never evaluate it,
    all other consumers share one evaluation."""
    from .wrapped_functions import LazyLayerNorm, force

    del lazy
    h = force(h)
    if isinstance(h, FwdLaplArray):
        return LazyLayerNorm(h, gamma, beta, eps, current_threshold())
    return _call('layer_norm', (h, gamma, beta), {'eps': eps})


def exp_envelope(d, sigma, pi):
    """``sum_I pi[I, o] exp(-sigma[I, o] d[..., I])``: exponential envelopes of orbitals from the
    electron-nucleus distances ``d (.., n_nuc)`` and constant ``sigma``, ``pi (n_nuc, O)`` (one
    fused rule; same result as the chain of primitives)."""
    return _call('exp_envelope', (d, sigma, pi))


def _tr(a, perm):
    """transpose that leaves an identity permutation (and a constant's laziness) alone"""
    perm = [int(i) for i in perm]
    if perm == list(range(len(perm))):
        return a
    return transpose(a, perm) if _is_triplet(a) else np.transpose(np.asarray(a), perm)


def _rs(a, shape):
    shape = tuple(int(n) for n in shape)
    if _shape(a) == shape:
        return a
    return reshape(a, shape) if _is_triplet(a) else np.reshape(np.asarray(a), shape)


def dot_general(lhs, rhs, dimension_numbers):
    """``jax.lax.dot_general``: ``dimension_numbers = ((lhs_contract, rhs_contract), (lhs_batch,
    rhs_batch))``, output axes ordered batch, lhs free, rhs free.  Either operand (or both) may
    carry derivatives, any axes may be contracted and a constant operand may have batch axes
    (per-head weights), as in ``_dot_general_one_constant`` and ``dot_general`` of the reference
    (folx/wrapped_functions.py:71-171, :174-309).

    Lowering.  One constant operand without batch axes: the operand with derivatives is brought
    to ``(free..., contract)`` and meets the constant as one matrix through ``dot`` (so the bias /
    activation / LayerNorm fusions still apply).  One constant operand with batch axes: one
    batched product ``(batch, i, k) x (batch, k, j)`` whose constant side is read once per batch
    element.  Two operands with derivatives: the batched two-operand rule through ``matmul``."""
    (lc, rc), (lb, rb) = dimension_numbers
    sl, sr = _shape(lhs), _shape(rhs)
    lc, lb = [int(i) % len(sl) for i in lc], [int(i) % len(sl) for i in lb]
    rc, rb = [int(i) % len(sr) for i in rc], [int(i) % len(sr) for i in rb]
    assert len(lc) == len(rc) and len(lb) == len(rb), dimension_numbers
    assert [sl[i] for i in lc] == [sr[i] for i in rc] and [sl[i] for i in lb] == [sr[i] for i in rb], \
        f'dot_general: {sl} and {sr} do not match under {dimension_numbers}'
    lf = [i for i in range(len(sl)) if i not in lc and i not in lb]
    rf = [i for i in range(len(sr)) if i not in rc and i not in rb]
    size = lambda shp, idx: int(np.prod([shp[i] for i in idx], dtype=np.int64))
    bshape = [sl[i] for i in lb]
    lshape, rshape = [sl[i] for i in lf], [sr[i] for i in rf]
    Bt, I, J, Kc = size(sl, lb), size(sl, lf), size(sr, rf), size(sl, lc)
    tl, trr = _is_triplet(lhs), _is_triplet(rhs)
    if isinstance(lhs, BatchedArray) or isinstance(rhs, BatchedArray):
        raise NotImplementedError('dot_general on walker-varying constants')
    if not tl and not trr:
        y = np.matmul(np.transpose(np.asarray(lhs), lb + lf + lc).reshape(*bshape, I, Kc),
                      np.transpose(np.asarray(rhs), rb + rc + rf).reshape(*bshape, Kc, J))
        return y.reshape(*bshape, *lshape, *rshape)
    if tl and trr:
        y = matmul(_rs(_tr(lhs, lb + lf + lc), (*bshape, I, Kc)), _rs(_tr(rhs, rb + rc + rf), (*bshape, Kc, J)))
        return _rs(y, (*bshape, *lshape, *rshape))
    # exactly one operand carries derivatives: h; the other one is the constant W
    h, hb, hf, hc, hshape = (lhs, lb, lf, lc, lshape) if tl else (rhs, rb, rf, rc, rshape)
    W, Wb, Wf, Wc, Wshape = (rhs, rb, rf, rc, rshape) if tl else (lhs, lb, lf, lc, lshape)
    Ih, Jw = (I, J) if tl else (J, I)
    W = np.asarray(W)
    if not hb:
        Wm = np.transpose(W, Wc + Wf).reshape(Kc, Jw)
        y = dot(_rs(_tr(h, hf + hc), (*hshape, Kc)), Wm)
        y = _rs(y, (*hshape, *Wshape))
        nh, nw = len(hshape), len(Wshape)
        return y if tl else _tr(y, [*range(nh, nh + nw), *range(nh)])
    Wm = np.transpose(W, Wb + Wc + Wf).reshape(Bt, Kc, Jw)
    y = _call('dot_general', (_rs(_tr(h, hb + hf + hc), (Bt, Ih, Kc)), Wm), {'batched_const': True})
    y = _rs(y, (*bshape, *hshape, *Wshape))
    nb, nh, nw = len(bshape), len(hshape), len(Wshape)
    return y if tl else _tr(y, [*range(nb), *range(nb + nh, nb + nh + nw), *range(nb, nb + nh)])


def matmul(a, b):
    """``numpy.matmul``: 1-D operands are vectors, leading axes broadcast against each other.
    Either operand may be a constant of any rank (a matrix, a vector, per-head matrices)."""
    ta, tb = _is_triplet(a), _is_triplet(b)
    if not ta and not tb:
        return np.matmul(a, b)
    if ta and not tb and np.ndim(b) == 2:
        return dot(a, b)                          # the plain layer: keeps every fusion of ``dot``
    if ta and tb:
        return _call('dot_general', (a, b), {})
    sa, sb = _shape(a), _shape(b)
    a_vec, b_vec = len(sa) == 1, len(sb) == 1
    la, lb_ = list(sa[:-2]) if not a_vec else [], list(sb[:-2]) if not b_vec else []
    L = max(len(la), len(lb_))
    # leading axes, right-aligned: both present and equal -> batch; one absent or of size 1 -> free axis of the other
    a_lead, b_lead, kinds = [], [], []
    for pos in range(L):
        ia_, ib_ = pos - (L - len(la)), pos - (L - len(lb_))
        na = la[ia_] if ia_ >= 0 else None
        nb = lb_[ib_] if ib_ >= 0 else None
        if na is not None and nb is not None and na == nb:
            kinds.append('batch'); a_lead.append(na); b_lead.append(nb)
        elif nb is None or (nb == 1 and na is not None):
            kinds.append('a'); a_lead.append(na)
        elif na is None or na == 1:
            kinds.append('b'); b_lead.append(nb)
        else:
            raise ValueError(f'matmul: shapes {sa} and {sb} do not broadcast')
    a2 = _rs(a, (*a_lead, *sa[(-1 if a_vec else -2):]))   # size-1 axes that only broadcast are dropped
    b2 = _rs(b, (*b_lead, *sb[(-1 if b_vec else -2):]))
    na_, nb_ = len(a_lead), len(b_lead)
    a_pos = iter(range(na_))
    b_pos = iter(range(nb_))
    axes_a, axes_b = {}, {}
    for pos, kind in enumerate(kinds):
        if kind in ('batch', 'a'):
            axes_a[pos] = next(a_pos)
        if kind in ('batch', 'b'):
            axes_b[pos] = next(b_pos)
    batch = [pos for pos, kind in enumerate(kinds) if kind == 'batch']
    dn = (([len(_shape(a2)) - 1], [nb_ if not b_vec else nb_]),
          ([axes_a[pos] for pos in batch], [axes_b[pos] for pos in batch]))
    y = dot_general(a2, b2, dn)
    # dot_general's order: batch, a's free axes (leads, i), b's free axes (leads, j)
    order = [('lead', pos) for pos in batch]
    order += [('lead', pos) for pos, kind in enumerate(kinds) if kind == 'a'] + ([] if a_vec else [('i', 0)])
    order += [('lead', pos) for pos, kind in enumerate(kinds) if kind == 'b'] + ([] if b_vec else [('j', 0)])
    want = [('lead', pos) for pos in range(L)] + ([] if a_vec else [('i', 0)]) + ([] if b_vec else [('j', 0)])
    return _tr(y, [order.index(t) for t in want])


def _einsum_pair(sa: str, sb: str, out: str, a, b):
    """One two-operand contraction as one ``dot_general``: indices shared by both operands and the output are
    batch axes, shared ones missing from the output are contracted, the others are the free axes of their
    operand -- the dimension numbers ``jnp.einsum`` hands to ``dot_general`` (folx/wrapped_functions.py:174-309)."""
    for idx, t in ((sa, a), (sb, b)):  # indices of one operand only that the output drops are summed first
        drop = [i for i, c in enumerate(idx) if c not in out and c not in (sb if idx is sa else sa)]
        if drop:
            red = sum(t, axis=tuple(drop)) if _is_triplet(t) else np.sum(np.asarray(t), axis=tuple(drop))
            kept = ''.join(c for i, c in enumerate(idx) if i not in drop)
            if idx is sa:
                a, sa = red, kept
            else:
                b, sb = red, kept
    batch = [c for c in sa if c in sb and c in out]
    contract = [c for c in sa if c in sb and c not in out]
    fa = [c for c in sa if c not in sb]
    fb = [c for c in sb if c not in sa]
    dn = (([sa.index(c) for c in contract], [sb.index(c) for c in contract]),
          ([sa.index(c) for c in batch], [sb.index(c) for c in batch]))
    y = dot_general(a, b, dn)
    cur = batch + fa + fb
    return _tr(y, [cur.index(c) for c in out])


def einsum(subscripts: str, *operands):
    """``numpy.einsum`` for any number of operands, with or without ``->`` and with ``...`` (an ellipsis stands for
    the same leading axes in every operand that has it): operands are contracted pairwise from the left, as
    ``jnp.einsum`` lowers them to a chain of ``dot_general`` (test/test_layers.py:255-262 uses
    ``'...i,...j,...ijk->...k'``).  No repeated index inside one operand."""
    spec = subscripts.replace(' ', '')
    ins, arrow, out = spec.partition('->')
    terms = ins.split(',')
    assert len(terms) == len(operands), f'einsum: {len(terms)} terms for {len(operands)} operands'
    ranks = [len(_shape(t)) for t in operands]
    n_ell = [r - (len(t) - 3) if '...' in t else 0 for t, r in zip(terms, ranks)]
    pool = [c for c in 'ABCDEFGHIJKLMNOPQRSTUVWXYZ' if c not in spec]
    width = max(n_ell) if n_ell else 0
    ell = ''.join(pool[:width])
    terms = [t.replace('...', ell[width - n:] if n else '') for t, n in zip(terms, n_ell)]
    if arrow:
        out = out.replace('...', ell)
    else:           # implicit form: the ellipsis axes, then every index that appears exactly once, in alphabetical order
        joined = ''.join(terms)
        out = ell + ''.join(sorted(c for c in set(joined) if joined.count(c) == 1 and c not in ell))
    for t, r in zip(terms, ranks):
        assert len(t) == r and len(set(t)) == len(t), f'einsum: term {t!r} for an operand of rank {r}'
    cur, scur = operands[0], terms[0]
    for k in range(1, len(operands)):
        later = set(out).union(*terms[k + 1:]) if k + 1 < len(terms) else set(out)
        mid = ''.join(dict.fromkeys(c for c in scur + terms[k] if c in later))
        cur, scur = _einsum_pair(scur, terms[k], mid, cur, operands[k]), mid
    drop = tuple(i for i, c in enumerate(scur) if c not in out)
    if drop:
        cur = sum(cur, axis=drop) if _is_triplet(cur) else np.sum(np.asarray(cur), axis=drop)
        scur = ''.join(c for c in scur if c in out)
    return _tr(cur, [scur.index(c) for c in out])


def softmax(a, axis=-1):
    """``jax.nn.softmax``: the shift by the maximum is a constant (stop_gradient), then exp, sum
    and div through their rules."""
    e = exp(subtract(a, amax_const(a, axis, keepdims=True)))
    return divide(e, sum(e, axis, keepdims=True))


def slogdet(A, row_axis=None, factor=None):
    """``numpy.linalg.slogdet`` over the last two axes; ``row_axis`` names another axis as the
    one holding the matrix rows (columns stay on the last axis, all other axes are batch axes
    in their order), which reads e.g. a dense layer's output (electron, determinant, orbital)
    in place.  ``factor`` (same shape as ``A``): the matrices are ``A * factor``; orbitals times
    envelopes are then multiplied while the matrices are loaded.  Same result as
    ``slogdet(multiply(A, factor))``."""
    from .wrapped_functions import LazyMul, LazyTranspose

    if isinstance(A, LazyTranspose) and row_axis is None and factor is None:
        A, row_axis = A.a, A.row_axis       # matrix rows on another axis: read in place
    if isinstance(A, LazyMul) and factor is None:
        A, factor = A.a, A.b                # slogdet(A * F): the product is formed while the matrices are loaded
    return _call('slogdet', (A,), {'row_axis': row_axis, 'factor': factor})


def det(A):
    return _call('det', (A,))


def minimum(a, b):
    return _call('min', (a, b))


def maximum(a, b):
    return _call('max', (a, b))


_SCATTER_KEYS = {'set': 'scatter', 'add': 'scatter-add', 'min': 'scatter_min', 'max': 'scatter_max'}


def scatter(operand, idx, updates, mode='set'):
    """``operand.at[idx].set / add / min / max(updates)`` (the ``mode``) for a static numpy
    index; either argument may be a constant.  Out-of-range integer indices drop their
    update."""
    return _call(_SCATTER_KEYS[mode], (operand, updates), {'idx': idx})


def inv(A):
    """``numpy.linalg.inv`` of a stack of matrices carrying derivatives."""
    return _call('inv', (A,))


def solve(A, b):
    """``numpy.linalg.solve``: ``b`` of rank 1 is a vector, else a stack of matrices; either
    operand may be a constant."""
    return _call('solve', (A, b))


def multi_head_self_attention(q, k, v, mask=None, input_mask=None, bias=None, **kwargs):
    """softmax(q k^T (+ bias)) v over per-walker arrays (n, H, d); no 1/sqrt(d) inside;
    ``bias`` is an optional edge-bias triplet (n, H, n).  Same registry keys as the
    reference's jitted wrappers (folx/experimental/pallas/attention/__init__.py:17-80)."""
    if bias is not None:
        return _call('_multi_head_self_edge_attention', (q, k, bias, v, mask, input_mask), kwargs)
    return _call('_multi_head_self_attention', (q, k, v, mask, input_mask), kwargs)


# reductions --------------------------------------------------------------------------------
def _axes(axis, nd):
    if axis is None:
        return tuple(range(nd))
    if isinstance(axis, int):
        axis = (axis,)
    return tuple(a % nd for a in axis)


def sum(a, axis=None, keepdims=False, window=None, scale=None):
    """``window = (lo, hi)`` with a single ``axis``: the sum of ``a[..., lo:hi, ...]`` along that
    axis, without forming the slice (what ``sum(a[..., lo:hi, ...], axis)`` becomes by itself).
    ``scale``: a constant factor applied in the same rule (the ``1 / n`` of ``mean``)."""
    from .wrapped_functions import LazySlice

    if isinstance(a, LazySlice) and window is None and _axes(axis, a.ndim) == (a.axis,):
        a, window = a.a, (a.lo, a.hi)       # the sum of a slice along the reduced axis: read in place
    shape = _shape(a)
    axes = _axes(axis, len(shape))
    if window is not None and not _is_triplet(a):
        a = getitem(a, tuple(slice(*window) if i == axes[0] else slice(None) for i in range(axes[0] + 1)))
        window = None
    kw = {'axes': axes}
    if window is not None:
        kw['window'] = tuple(window)
    if scale is not None:
        kw['scale'] = float(scale)
    out = _call('reduce_sum', (a,), kw)
    if keepdims:
        out = reshape(out, tuple(1 if i in axes else n for i, n in enumerate(shape)))
    return out


def mean(a, axis=None, keepdims=False, window=None):
    shape = _shape(a)
    axes = _axes(axis, len(shape))
    n = int(np.prod([shape[i] for i in axes], dtype=int)) if window is None else int(window[1] - window[0])
    return sum(a, axis, keepdims, window, scale=1.0 / n)


def amax_const(a, axis, keepdims=False):
    """max of the values as a derivative-free array (``stop_gradient(max(a))``)."""
    shape = _shape(a)
    axes = _axes(axis, len(shape))
    out = _call('reduce_max_values', (a,), {'axes': axes})
    if keepdims:
        out = reshape(out, tuple(1 if i in axes else n for i, n in enumerate(shape)))
    return out


def logsumexp(a, axis=-1, b=None):
    """``jax.nn.logsumexp(a, axis, b=b, return_sign=True)``: the same primitive sequence
    (max shift under stop_gradient, exp, weighted sum, log|.|).  Returns (value, sign)."""
    m = amax_const(a, axis, keepdims=True)
    e = exp(subtract(a, m))
    if b is not None:
        e = multiply(e, b)
    s = sum(e, axis)
    sg = sign(s)
    val = add(log(abs(s)), reshape(m, _shape(s)))
    return val, sg


# indexing ----------------------------------------------------------------------------------
def reshape(a, shape):
    shape = tuple(int(s) for s in shape)
    if -1 in shape:
        tot = int(np.prod(_shape(a), dtype=int))
        rest = -int(np.prod(shape, dtype=int))
        shape = tuple(tot // rest if s == -1 else s for s in shape)
    from .wrapped_functions import LazyDot

    if (isinstance(a, LazyDot) and a._value is None and len(shape) >= 1 and shape[-1] == a.shape[-1]
            and isinstance(a.h, FwdLaplArray) and a.kwargs.get('row_slice') is None and a.kwargs.get('norm') is None):
        # only the leading axes change: the same product on the input with those leading axes, its epilogue
        # (bias, activation, skip connection) still open -- e.g. `(h.reshape(-1, K) @ W).reshape(n, n, N) + b`
        h = _call('reshape', (a.h,), {'new_sizes': (*shape[:-1], a.h.shape[-1])})
        return LazyDot(h, a.W, a.kwargs, shape, a.thr)
    return _call('reshape', (a,), {'new_sizes': shape})


def transpose(a, axes=None):
    from .wrapped_functions import LazyMul, LazyTranspose

    nd = len(_shape(a))
    axes = tuple(range(nd))[::-1] if axes is None else tuple(ax % nd for ax in axes)
    if nd >= 3 and isinstance(a, (FwdLaplArray, LazyMul)) and axes[-1] == nd - 1 and axes[-2] != nd - 2 \
            and list(axes[:-2]) == [i for i in range(nd - 1) if i != axes[-2]]:
        return LazyTranspose(a, axes, current_threshold())  # one axis moved in front of the last: slogdet reads it in place
    return _call('transpose', (a,), {'permutation': axes})


def swapaxes(a, i, j):
    nd = len(_shape(a))
    axes = list(range(nd))
    axes[i % nd], axes[j % nd] = axes[j % nd], axes[i % nd]
    return transpose(a, axes)


def expand_dims(a, axis):
    shape = list(_shape(a))
    axis = axis % (len(shape) + 1)
    shape.insert(axis, 1)
    return reshape(a, shape)


def squeeze(a, axis):
    shape = list(_shape(a))
    axis = axis % len(shape)
    assert shape[axis] == 1
    del shape[axis]
    return reshape(a, shape)


def broadcast_to(a, shape, lazy=True):
    """A vector broadcast along new leading axes is deferred: a concatenation that a product
    reads in parts takes it as it is, everything else evaluates it."""
    from .wrapped_functions import LazyBroadcast, force

    del lazy
    shape = tuple(int(n) for n in shape)
    a = force(a)
    if isinstance(a, FwdLaplArray) and a.ndim == 1 and len(shape) >= 2 and shape[-1] == a.shape[-1]:
        return LazyBroadcast(a, shape, current_threshold())  # a per-walker vector shown to every row
    src = _shape(a)
    off = len(shape) - len(src)
    return _call('broadcast_in_dim', (a,), {'shape': shape, 'broadcast_dimensions': tuple(range(off, len(shape)))})


def getitem(a, idx):
    from .wrapped_functions import LazySlice, force

    a = force(a)
    if isinstance(a, FwdLaplArray):
        # a contiguous window along ONE axis, everything else taken whole: deferred, so that the product
        # or the sum that reads it can take the window in place
        items = idx if isinstance(idx, tuple) else (idx,)
        if all(isinstance(i, slice) for i in items) and len(items) <= a.ndim:
            cut = [(ax, *i.indices(a.shape[ax])) for ax, i in enumerate(items)
                   if i.indices(a.shape[ax]) != (0, a.shape[ax], 1)]
            if len(cut) == 1 and cut[0][3] == 1 and cut[0][1] < cut[0][2]:
                return LazySlice(a, cut[0][0], cut[0][1], cut[0][2], current_threshold())
    return _call('slice', (a,), {'idx': idx})


def concatenate(arrs, axis=-1, lazy=True):
    """Along the last axis of triplets the result is deferred: a product that can read its operand
    in parts never forms the concatenation (nor the broadcasts among the parts)."""
    from .wrapped_functions import LazyBroadcast, LazyConcat, force

    del lazy
    arrs = tuple(t if isinstance(t, LazyBroadcast) else force(t) for t in arrs)
    nd = len(_shape(arrs[0]))
    if axis % nd == nd - 1 and nd >= 2 and len(arrs) > 1 and all(isinstance(t, (FwdLaplArray, LazyBroadcast)) for t in arrs) \
            and all(tuple(t.shape[:-1]) == tuple(arrs[0].shape[:-1]) for t in arrs):
        return LazyConcat(arrs, current_threshold())
    return _call('concatenate', arrs, {'dimension': axis})


# composed rules ---------------------------------------------------------------------------
def clip(a, lo=None, hi=None):
    """``numpy.clip`` with constant bounds (``jax.lax.clamp``): min / max against constants."""
    out = a
    if hi is not None:
        out = minimum(out, hi)
    if lo is not None:
        out = maximum(out, lo)
    return out


def where(cond, a, b):
    """``numpy.where`` with a derivative-free condition (``select_n``): linear in a and b."""
    c = cond.data.to(dtype=cond.data.dtype).float() if isinstance(cond, BatchedArray) else \
        np.asarray(cond, dtype=np.float32)
    ci = BatchedArray(1.0 - c) if isinstance(cond, BatchedArray) else (1.0 - c)
    cc = BatchedArray(c) if isinstance(cond, BatchedArray) else c
    return add(multiply(a, cc), multiply(b, ci))


def cumsum(a, axis=-1):
    """Cumulative sum along one axis: a product with a triangular matrix of ones (LINEAR)."""
    nd = len(_shape(a))
    ax = axis % nd
    n = _shape(a)[ax]
    tri = np.triu(np.ones((n, n), dtype=np.float32))
    if ax == nd - 1:
        return dot(a, tri)
    return swapaxes(dot(swapaxes(a, ax, -1), tri), ax, -1)


def _fold(op, a, axis):
    """Reduction of one axis by a binary rule, as a tree: the two halves of the axis are combined element
    by element (one launch of the binary rule per level, log2(n) levels), a leftover middle entry rides
    along -- any length of the axis."""
    nd = len(_shape(a))
    ax = axis % nd
    part = lambda t, lo, hi: getitem(t, tuple(slice(lo, hi) if d == ax else slice(None) for d in range(nd)))
    n = _shape(a)[ax]
    assert n >= 1, 'reduction of an empty axis'
    while n > 1:
        h = n // 2
        folded = op(part(a, 0, h), part(a, h, 2 * h))
        a = folded if n == 2 * h else concatenate([folded, part(a, 2 * h, n)], axis=ax)
        n = h + (n - 2 * h)
    return squeeze(a, ax)


def amax(a, axis=-1):
    """max along an axis with derivatives (``reduce_max``): pairwise ``maximum`` over the axis."""
    return _fold(maximum, a, axis)


def amin(a, axis=-1):
    return _fold(minimum, a, axis)


def prod(a, axis=-1):
    """Product along an axis (``reduce_prod``): pairwise ``multiply`` over the axis."""
    return _fold(multiply, a, axis)


def flip(a, axis):
    nd = len(_shape(a))
    axes = (axis,) if np.isscalar(axis) else tuple(axis)
    return _call('rev', (a,), {'dimensions': tuple(ax % nd for ax in axes)})


def pad(a, pad_width, constant_values=0.0):
    """``numpy.pad`` (constant mode): concatenation with constant blocks (``lax.pad``)."""
    shape = list(_shape(a))
    pw = [tuple(p) for p in pad_width] if np.ndim(pad_width) == 2 else [tuple(pad_width)] * len(shape)
    out = a
    for ax, (lo, hi) in enumerate(pw):
        parts = []
        if lo:
            parts.append(np.full((*shape[:ax], lo, *shape[ax + 1:]), constant_values, dtype=np.float32))
        parts.append(out)
        if hi:
            parts.append(np.full((*shape[:ax], hi, *shape[ax + 1:]), constant_values, dtype=np.float32))
        if len(parts) > 1:
            out = concatenate(parts, axis=ax)
        shape[ax] += lo + hi
    return out


def lax_pad(operand, padding_value, padding_config):
    """``jax.lax.pad`` (the ``pad_p`` primitive, folx/wrapped_functions.py:480-487): per axis ``(low, high, interior)``
    with negative ``low`` / ``high`` cropping the (interior-padded) array, and a padding value that may itself carry
    derivatives.  Every output element is an operand element or the padding value, so the result is one static
    position gather from ``[operand elements..., padding value]``; sparse Jacobians stay sparse."""
    shape = tuple(_shape(operand))
    cfg = [tuple(int(v) for v in c) for c in padding_config]
    assert len(cfg) == len(shape), 'lax_pad: one (low, high, interior) per axis'
    n_total = int(np.prod(shape)) if shape else 1
    per_axis = []
    for n, (lo, hi, it) in zip(shape, cfg):
        assert it >= 0, 'lax_pad: negative interior padding'
        dil = n + max(n - 1, 0) * it
        m = np.full(max(lo + dil + hi, 0), -1, dtype=np.int64)
        pos = lo + np.arange(n) * (it + 1)
        ok = (pos >= 0) & (pos < m.size)
        m[pos[ok]] = np.arange(n)[ok]
        per_axis.append(m)
    grids = np.meshgrid(*per_axis, indexing='ij') if per_axis else []
    valid = np.ones([m.size for m in per_axis], dtype=bool)
    for g in grids:
        valid &= g >= 0
    table = np.full(valid.shape, n_total, dtype=np.int64)      # n_total: the slot of the padding value
    if valid.any():
        table[valid] = np.ravel_multi_index(tuple(g[valid] for g in grids), shape)
    pv = padding_value if _is_triplet(padding_value) else np.full((1,), float(np.asarray(padding_value)), dtype=np.float32)
    src = concatenate([reshape(operand, (n_total,)), reshape(pv, (1,))], axis=0)
    return getitem(src, table)


floor, ceil, round = (lambda a: _call('floor', (a,))), (lambda a: _call('ceil', (a,))), (lambda a: _call('round', (a,)))
greater, greater_equal = (lambda a, b: _call('gt', (a, b))), (lambda a, b: _call('ge', (a, b)))
less, less_equal = (lambda a, b: _call('lt', (a, b))), (lambda a, b: _call('le', (a, b)))
equal, not_equal = (lambda a, b: _call('eq', (a, b))), (lambda a, b: _call('ne', (a, b)))


trunc, isfinite = (lambda a: _call('trunc', (a,))), (lambda a: _call('is_finite', (a,)))
logical_and, logical_or = (lambda a, b: _call('and', (a, b))), (lambda a, b: _call('or', (a, b)))
logical_xor, logical_not = (lambda a, b: _call('xor', (a, b))), (lambda a: _call('not', (a,)))


def argmax(a, axis=-1):
    """Index of the maximum along ``axis`` (no derivatives)."""
    return _call('argmax', (a,), {'axis': axis % len(_shape(a))})


def argmin(a, axis=-1):
    return _call('argmin', (a,), {'axis': axis % len(_shape(a))})


def exp2(a):
    return exp(multiply(a, np.float32(np.log(2.0))))


def remainder(a, b):
    """C-style remainder ``a - b trunc(a / b)`` (``jax.lax.rem``): the quotient is piecewise
    constant, so the rule is linear in a and b."""
    return subtract(a, multiply(b, trunc(divide(a, b))))


fmod = remainder


def arctan2(y, x):
    """``atan2(y, x)`` from the two half-plane formulas ``atan(y / x) (+- pi)`` for
    ``|x| >= |y|`` and ``+-pi/2 - atan(x / y)`` otherwise.  The denominator of the branch
    that is not taken is replaced by 1 before the division, so no infinity or NaN of a dead
    branch reaches the result."""
    big = greater_equal(abs(stop_gradient(x)), abs(stop_gradient(y)))     # |x| >= |y|
    xs, ys = where(big, x, 1.0), where(big, 1.0, y)
    ypos = greater_equal(stop_gradient(y), 0.0)
    xneg = less(stop_gradient(x), 0.0)
    pi = np.float32(np.pi)
    sgn = subtract(multiply(ypos, 2.0), 1.0)                                # +1 for y >= 0, else -1
    off_a = multiply(multiply(xneg, sgn), pi)                               # +-pi on the left half plane
    branch_a = add(arctan(divide(y, xs)), off_a)
    branch_b = subtract(multiply(sgn, pi / 2), arctan(divide(x, ys)))
    return where(big, branch_a, branch_b)


def split(a, indices_or_sections, axis=0):
    """``numpy.split``: equal sections or explicit cut points along ``axis``."""
    nd = len(_shape(a))
    ax = axis % nd
    n = _shape(a)[ax]
    if np.isscalar(indices_or_sections):
        k = int(indices_or_sections)
        assert n % k == 0, 'array split does not result in an equal division'
        cuts = [i * (n // k) for i in range(k + 1)]
    else:
        cuts = [0, *[int(c) for c in indices_or_sections], n]
    return [getitem(a, tuple(slice(lo, hi) if d == ax else slice(None) for d in range(nd)))
            for lo, hi in zip(cuts[:-1], cuts[1:])]


def stack(arrs, axis=0):
    arrs = list(arrs)
    nd = len(_shape(arrs[0])) + 1
    return concatenate([expand_dims(t, axis % nd) for t in arrs], axis=axis % nd)


def unstack(a, axis=0):
    return [squeeze(t, axis) for t in split(a, _shape(a)[axis % len(_shape(a))], axis)]


def tile(a, reps):
    reps = (reps,) if np.isscalar(reps) else tuple(reps)
    nd = max(len(reps), len(_shape(a)))
    reps = (1,) * (nd - len(reps)) + tuple(int(r) for r in reps)
    out = reshape(a, (1,) * (nd - len(_shape(a))) + tuple(_shape(a)))
    for ax, r in enumerate(reps):
        if r > 1:
            out = concatenate([out] * r, axis=ax)
    return out


def copy(a):
    return a


real = conj = copy      # real arithmetic only: the complex rules of the reference have no use here


def imag(a):
    return multiply(a, 0.0)


def astype(a, dtype):
    """float32 is the only arithmetic type of the path; integer / boolean targets give values
    without derivatives (``convert_element_type``, folx/wrapped_functions.py:313-352)."""
    if np.issubdtype(np.dtype(dtype), np.floating):
        return a
    return trunc(a) if np.issubdtype(np.dtype(dtype), np.integer) else not_equal(a, 0.0)


def dynamic_slice(a, start_indices, slice_sizes):
    """``jax.lax.dynamic_slice`` for start indices known at trace time (clamped like lax)."""
    shape = _shape(a)
    idx = []
    for s0, sz, n in zip(start_indices, slice_sizes, shape):
        s0 = int(np.clip(int(s0), 0, n - int(sz)))
        idx.append(slice(s0, s0 + int(sz)))
    return getitem(a, tuple(idx))


def dynamic_update_slice(a, update, start_indices):
    """``jax.lax.dynamic_update_slice`` for start indices known at trace time: linear in both
    operands (a zero-padded update blended in with a 0/1 mask)."""
    shape, ushape = _shape(a), _shape(update)
    widths, mask = [], np.zeros(shape, dtype=np.float32)
    sl = []
    for s0, un, n in zip(start_indices, ushape, shape):
        s0 = int(np.clip(int(s0), 0, n - un))
        widths.append((s0, n - un - s0))
        sl.append(slice(s0, s0 + un))
    mask[tuple(sl)] = 1.0
    return add(multiply(a, 1.0 - mask), pad(update, widths))


def logaddexp(a, b):
    """log(exp a + exp b) = a + softplus(b - a)."""
    return add(a, softplus(subtract(b, a)))


def _scan(op, a, axis):
    """Inclusive scan of one axis by an associative binary rule in log2(n) levels: at level s every entry
    i >= s is combined with entry i - s (one launch of the binary rule per level) -- any length of the axis."""
    nd = len(_shape(a))
    ax = axis % nd
    n = _shape(a)[ax]
    part = lambda t, lo, hi: getitem(t, tuple(slice(lo, hi) if d == ax else slice(None) for d in range(nd)))
    s_ = 1
    while s_ < n:
        a = concatenate([part(a, 0, s_), op(part(a, 0, n - s_), part(a, s_, n))], axis=ax)
        s_ *= 2
    return a


def cumprod(a, axis=-1):
    return _scan(multiply, a, axis)


def cummax(a, axis=-1):
    return _scan(maximum, a, axis)


def cummin(a, axis=-1):
    return _scan(minimum, a, axis)


def _composed(fn, *kw_names):
    """Registry rule ``(args, kwargs, sparsity_threshold)`` for a composed function, so that
    it is reachable under its primitive name like the kernel-backed rules."""

    def rule(args, kwargs, threshold):
        with sparsity_threshold(threshold):
            return fn(*args, **{k: kwargs[k] for k in kw_names if k in kwargs})

    rule.__name__ = fn.__name__
    return rule


# jax.numpy / jax.nn names that trace to chains of the primitives above in the reference; the same chains here
def relu(a):
    return maximum(a, 0.0)


def leaky_relu(a, negative_slope=0.01):
    return where(greater_equal(a, 0.0), a, multiply(a, float(negative_slope)))


def elu(a, alpha=1.0):
    return where(greater(a, 0.0), a, multiply(expm1(minimum(a, 0.0)), float(alpha)))


def gelu(a, approximate=True):
    """``jax.nn.gelu``: the tanh form by default, ``approximate=False`` the erf form (test/test_layers.py:709)."""
    if approximate:
        inner = multiply(add(a, multiply(integer_pow(a, 3), 0.044715)), float(np.sqrt(2.0 / np.pi)))
        return multiply(multiply(a, 0.5), add(tanh(inner), 1.0))
    return multiply(multiply(a, 0.5), add(erf(multiply(a, float(1.0 / np.sqrt(2.0)))), 1.0))


def log_softmax(a, axis=-1):
    shifted = subtract(a, amax_const(a, axis, keepdims=True))
    return subtract(shifted, log(sum(exp(shifted), axis, keepdims=True)))


def var(a, axis=None, keepdims=False):
    c = subtract(a, mean(a, axis, keepdims=True))
    return mean(square(c), axis, keepdims)


def std(a, axis=None, keepdims=False):
    return sqrt(var(a, axis, keepdims))


def norm(a, axis=None, keepdims=False):
    """``jnp.linalg.norm`` (2-norm of a vector / Frobenius norm over ``axis``)."""
    return sqrt(sum(square(a), axis, keepdims))


def vdot(a, b):
    """``jnp.vdot`` on real data: both arguments flattened, one number."""
    n = int(np.prod(_shape(a), dtype=int))
    return sum(multiply(reshape(a, (n,)), reshape(b, (n,))))


def inner(a, b):
    return tensordot(a, b, axes=((-1,), (-1,)))


def outer(a, b):
    na, nb = int(np.prod(_shape(a), dtype=int)), int(np.prod(_shape(b), dtype=int))
    return multiply(reshape(a, (na, 1)), reshape(b, (1, nb)))


def tensordot(a, b, axes=2):
    """``jnp.tensordot``: a ``dot_general`` without batch axes."""
    nda, ndb = len(_shape(a)), len(_shape(b))
    if isinstance(axes, int):
        ca, cb = tuple(range(nda - axes, nda)), tuple(range(axes))
    else:
        ca, cb = axes
        ca = (ca,) if isinstance(ca, int) else tuple(ca)
        cb = (cb,) if isinstance(cb, int) else tuple(cb)
    return dot_general(a, b, ((tuple(i % nda for i in ca), tuple(i % ndb for i in cb)), ((), ())))


def moveaxis(a, source, destination):
    nd = len(_shape(a))
    src = [s % nd for s in ((source,) if isinstance(source, int) else source)]
    dst = [d % nd for d in ((destination,) if isinstance(destination, int) else destination)]
    order = [i for i in range(nd) if i not in src]
    for d, s_ in sorted(zip(dst, src)):
        order.insert(d, s_)
    return transpose(a, order)


def take(a, indices, axis=None):
    """``jnp.take`` with static integer indices (out-of-range entries are an error, as under ``mode='raise'``)."""
    idx = np.asarray(indices)
    if axis is None:
        return getitem(reshape(a, (int(np.prod(_shape(a), dtype=int)),)), idx)
    axis = axis % len(_shape(a))
    return getitem(a, (*([slice(None)] * axis), idx))


def diagonal(a, offset=0):
    """Diagonal of the last two axes, as a new last axis (``jnp.diagonal(a, offset, -2, -1)``)."""
    n, m = _shape(a)[-2:]
    i = np.arange(max(min(n + min(offset, 0), m - max(offset, 0)), 0))
    nd = len(_shape(a))
    return getitem(a, (*([slice(None)] * (nd - 2)), i - min(offset, 0), i + max(offset, 0)))


def trace(a, offset=0):
    return sum(diagonal(a, offset), axis=-1)


def roll(a, shift, axis):
    n = _shape(a)[axis]
    return take(a, (np.arange(n) - int(shift)) % n, axis)


def repeat(a, repeats, axis):
    return take(a, np.repeat(np.arange(_shape(a)[axis]), int(repeats)), axis)


def zeros_like(a):
    return np.zeros(tuple(_shape(a)), dtype=np.float32)


def ones_like(a):
    return np.ones(tuple(_shape(a)), dtype=np.float32)


erfinv, gammaln = erf_inv, lgamma   # (jnp.max / jnp.min along one axis are amax / amin: the builtins keep their names here)


# jnp.linalg / jax.nn / jax.scipy.special spellings of the functions above
import types as _types

linalg = _types.SimpleNamespace(slogdet=slogdet, det=det, inv=inv, solve=solve, norm=norm)
nn = _types.SimpleNamespace(softmax=softmax, log_softmax=log_softmax, logsumexp=logsumexp, gelu=gelu, silu=silu, relu=relu,
                            elu=elu, leaky_relu=leaky_relu, sigmoid=sigmoid, softplus=softplus, tanh=tanh)
special = _types.SimpleNamespace(erf=erf, erfc=erfc, erfinv=erf_inv, gammaln=lgamma, digamma=digamma, logsumexp=logsumexp)


# primitive names of jax.lax (folx/wrapped_functions.py:376-399, :468-513)
register_function('clamp', lambda args, kw, thr: _composed(lambda lo, x, hi: clip(x, lo, hi))(args, kw, thr))
register_function('select_n', lambda args, kw, thr: _composed(lambda c, b, a: where(c, a, b))(args, kw, thr))
register_function('cumsum', _composed(cumsum, 'axis'))
register_function('reduce_max', _composed(amax, 'axis'))
register_function('reduce_min', _composed(amin, 'axis'))
register_function('reduce_prod', _composed(prod, 'axis'))
register_function('cumprod', _composed(cumprod, 'axis'))
register_function('cummax', _composed(cummax, 'axis'))
register_function('cummin', _composed(cummin, 'axis'))
register_function('logaddexp', _composed(logaddexp))
register_function('pad', lambda args, kw, thr: _composed(lax_pad, 'padding_config')(args, kw, thr) if 'padding_config' in kw
                  else _composed(pad, 'constant_values')(args, kw, thr))   # lax.pad_p.bind(operand, value, padding_config=...)
register_function('atan2', _composed(arctan2))                       # folx/wrapped_functions.py:419
register_function('rem', _composed(remainder))                       # :438
register_function('exp2', _composed(exp2))                           # :636
register_function('split', _composed(split, 'indices_or_sections', 'axis'))   # :628
register_function('stack', _composed(lambda *arrs, axis=0: stack(arrs, axis), 'axis'))     # :641
register_function('unstack', _composed(unstack, 'axis'))             # :651
register_function('tile', _composed(tile, 'reps'))                   # :660
register_function('copy', _composed(copy))                           # :638
register_function('squeeze', _composed(lambda a, dimensions: squeeze(a, dimensions[0]) if len(dimensions) == 1
                                       else reshape(a, [n for i, n in enumerate(_shape(a)) if i not in dimensions]),
                                       'dimensions'))                # :503
register_function('real', _composed(real))                           # :358
register_function('conj', _composed(conj))                           # :356
register_function('imag', _composed(imag))                           # :357
register_function('convert_element_type', _composed(lambda a, new_dtype=np.float32: astype(a, new_dtype), 'new_dtype'))
register_function('dynamic_slice', _composed(lambda a, *start, slice_sizes: dynamic_slice(a, start, slice_sizes),
                                             'slice_sizes'))          # :468
register_function('dynamic_update_slice', _composed(lambda a, u, *start: dynamic_update_slice(a, u, start)))  # :488


# constants, dtypes and tests on plain arrays are numpy's own (``jnp.zeros``, ``jnp.eye``, ``jnp.float32`` ...)
zeros, ones, eye, full, arange, linspace, array, asarray = (np.zeros, np.ones, np.eye, np.full, np.arange, np.linspace,
                                                            np.array, np.asarray)
float16, float32, float64, int8, int16, int32, int64, uint8, uint16, uint32, uint64, bool_ = (
    np.float16, np.float32, np.float64, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64,
    np.bool_)
rem = remainder                                      # jax.lax.rem


def full_like(a, fill_value, dtype=None):
    return np.full(_shape(a), fill_value, dtype=dtype or np.float32)


def convert_element_type(a, new_dtype):              # jax.lax.convert_element_type
    return astype(a, new_dtype)


def allclose(a, b, rtol=1e-5, atol=1e-8):
    """``numpy.allclose`` on values (triplets contribute their ``x``)."""
    from .wrapped_functions import force

    val = lambda v: force(v).x.detach().cpu().numpy() if _is_triplet(v) else (  # noqa: E731
        v.data.detach().cpu().numpy() if isinstance(v, BatchedArray) else np.asarray(v))
    return bool(np.allclose(val(a), val(b), rtol=rtol, atol=atol))


def _reduce_named(fold):
    def fn(a, axis=None, keepdims=False):
        shape = _shape(a)
        axes = sorted(_axes(axis, len(shape)), reverse=True)
        out = a
        for ax in axes:
            out = fold(out, axis=ax)
        if keepdims:
            out = reshape(out, tuple(1 if i in axes else n for i, n in enumerate(shape)))
        return out

    return fn


_LATE = {'max': _reduce_named(amax), 'min': _reduce_named(amin)}


def __getattr__(name):
    # ``fnp.max`` / ``fnp.min`` (``jnp.max``: all axes by default) without shadowing the builtins this module uses
    try:
        return _LATE[name]
    except KeyError:
        raise AttributeError(f'module {__name__!r} has no attribute {name!r}') from None


def fori_loop(lower, upper, body_fun, init_val):
    """``jax.lax.fori_loop`` with bounds known when the model is written: the loop simply runs (define-by-run), each
    iteration through the ordinary rules."""
    val = init_val
    for i in range(int(lower), int(upper)):
        val = body_fun(i, val)
    return val


def scan(f, init, xs=None, length=None, reverse=False):
    """``jax.lax.scan(f, init, xs)``: ``carry, y = f(carry, x)`` over the leading axis of ``xs`` -- constants, as in the
    reference (folx/interpreter.py:133-184 asserts that the scanned-over inputs carry no derivatives), or triplets
    (sliced through the indexing rule).  ``xs`` may be a tuple / list / dict of arrays or None (then ``length``
    iterations with ``x = None``).  The ``y`` of the iterations are stacked along a new leading axis; ``None`` stays None."""
    def lead(v):
        if isinstance(v, (tuple, list)):
            return lead(v[0])
        if isinstance(v, dict):
            return lead(next(iter(v.values())))
        return _shape(v)[0]

    def item(v, i):
        if isinstance(v, (tuple, list)):
            return type(v)(item(t, i) for t in v)
        if isinstance(v, dict):
            return {k: item(t, i) for k, t in v.items()}
        return getitem(v, i) if _is_triplet(v) or isinstance(v, BatchedArray) else np.asarray(v)[i]

    n = int(length) if xs is None else lead(xs)
    order = range(n - 1, -1, -1) if reverse else range(n)
    carry, ys = init, [None] * n
    for i in order:
        carry, ys[i] = f(carry, None if xs is None else item(xs, i))

    def pile(parts):
        first = parts[0]
        if first is None:
            return None
        if isinstance(first, (tuple, list)):
            return type(first)(pile([p[k] for p in parts]) for k in range(len(first)))
        if isinstance(first, dict):
            return {k: pile([p[k] for p in parts]) for k in first}
        if any(_is_triplet(p) or isinstance(p, BatchedArray) for p in parts):
            return stack(parts, axis=0)
        return np.stack([np.asarray(p) for p in parts], axis=0)

    return carry, (pile(ys) if n > 0 else None)

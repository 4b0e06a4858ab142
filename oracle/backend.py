"""Whole-model oracle: the operator namespace of ``folx_amd.numpy`` on numpy arrays with
dense Jacobians (test infrastructure; also the CPU baseline timed by ``bench.py``).

A model written against the namespace (``xp.dot``, ``xp.tanh``, ``xp.slogdet`` ...) runs
unchanged on this backend.  Values are ``OArr`` triplets in the package layout
``x (B, *s)``, ``J (P, B, *s)``, ``lap (B, *s)``; walker-varying constants are ``OConst``
(data ``(B, *s)``); walker-invariant constants are plain numpy arrays / scalars of the
logical shape ``s``.  Every op applies the rule from ``oracle.rules``.
"""

from __future__ import annotations

import numpy as np
from builtins import sum as builtins_sum

from . import rules


class OConst:
    """A constant that differs per walker: data (B, *s)."""

    def __init__(self, data):
        self.data = np.asarray(data)

    @property
    def shape(self):
        return self.data.shape[1:]


class OArr:
    def __init__(self, x, J, lap):
        self.x, self.J, self.lap = x, J, lap

    @property
    def shape(self):
        return self.x.shape[1:]

    @property
    def ndim(self):
        return self.x.ndim - 1

    @property
    def B(self):
        return self.x.shape[0]

    @property
    def P(self):
        return self.J.shape[0]

    # operator sugar -----------------------------------------------------------------
    def __add__(self, o):
        return add(self, o)

    __radd__ = __add__

    def __sub__(self, o):
        return subtract(self, o)

    def __rsub__(self, o):
        return subtract(o, self)

    def __mul__(self, o):
        return multiply(self, o)

    __rmul__ = __mul__

    def __truediv__(self, o):
        return divide(self, o)

    def __neg__(self):
        return negative(self)

    def __getitem__(self, idx):
        return getitem(self, idx)

    def reshape(self, *shape):
        if len(shape) == 1 and isinstance(shape[0], (tuple, list)):
            shape = tuple(shape[0])
        return reshape(self, shape)

    def sum(self, axis=None, keepdims=False):
        return sum(self, axis, keepdims)


def init_state(x, weights=None, dtype=None) -> OArr:
    """x (B, *s) -> J = identity rows (folx/interpreter.py:295), lap = 0 (:297)."""
    x = np.asarray(x, dtype=dtype)
    B = x.shape[0]
    n = int(np.prod(x.shape[1:], dtype=int))
    eye = np.eye(n, dtype=x.dtype)
    if weights is not None:
        eye = eye * np.broadcast_to(np.asarray(weights, dtype=x.dtype), x.shape[1:]).reshape(-1)
    J = np.broadcast_to(eye.reshape(n, 1, *x.shape[1:]), (n, B, *x.shape[1:])).copy()
    return OArr(x, J, np.zeros_like(x))


def _is(a):
    return isinstance(a, OArr)


def _const(c, like: OArr):
    """Constant as (array (B or 1, *s_c), logical ndim)."""
    dt = like.x.dtype
    if isinstance(c, OConst):
        d = c.data.astype(dt)
        return d, d.ndim - 1
    c = np.asarray(c, dtype=dt)
    return c[None], c.ndim


def _pad(t: OArr, nd: int) -> OArr:
    """Prepend size-1 logical axes so the triplet has ``nd`` logical dims."""
    ex = nd - t.ndim
    if ex <= 0:
        return t
    B, P = t.B, t.P
    one = [1] * ex
    return OArr(
        t.x.reshape(B, *one, *t.shape),
        t.J.reshape(P, B, *one, *t.shape),
        t.lap.reshape(B, *one, *t.shape),
    )


def _padJ(a: OArr, b: OArr):
    """Dense Jacobians of different row counts are zero-extended (folx/utils.py:432-450)."""
    P = max(a.P, b.P)

    def ext(J):
        if J.shape[0] == P:
            return J
        z = np.zeros((P - J.shape[0], *J.shape[1:]), dtype=J.dtype)
        return np.concatenate([J, z], 0)

    return ext(a.J), ext(b.J)


def _bcast3(a: OArr, b: OArr):
    nd = max(a.ndim, b.ndim)
    a, b = _pad(a, nd), _pad(b, nd)
    Ja, Jb = _padJ(a, b)
    xa, xb = np.broadcast_arrays(a.x, b.x)
    Ja, Jb = np.broadcast_arrays(Ja, Jb)
    La, Lb = np.broadcast_arrays(a.lap, b.lap)
    return (xa, Ja, La), (xb, Jb, Lb)


def _with_const(a: OArr, c):
    """Align a triplet and a constant: returns (padded triplet, constant (B|1, *s))."""
    c, cn = _const(c, a)
    nd = max(a.ndim, cn)
    a = _pad(a, nd)
    c = c.reshape(c.shape[0], *([1] * (nd - cn)), *c.shape[1:])
    return a, c


def add(a, b, sign=1.0):
    if _is(a) and _is(b):
        ta, tb = _bcast3(a, b)
        return OArr(*rules.add_rule(*ta, *tb, sign=sign))
    if _is(a):
        a, c = _with_const(a, b)
        x = a.x + sign * c
        return OArr(
            x,
            np.broadcast_to(a.J, (a.P, *x.shape)).copy(),
            np.broadcast_to(a.lap, x.shape).copy(),
        )
    # constant +- triplet
    return add(multiply(b, sign), a, 1.0)


def subtract(a, b):
    return add(a, b, sign=-1.0)


def multiply(a, b):
    if not _is(a) and not _is(b):
        da = a.data if isinstance(a, OConst) else np.asarray(a)[None]
        db = b.data if isinstance(b, OConst) else np.asarray(b)[None]
        return OConst(da * db)
    if _is(a) and _is(b):
        ta, tb = _bcast3(a, b)
        return OArr(*rules.mul_rule(*ta, *tb))
    if _is(b):
        a, b = b, a
    a, c = _with_const(a, b)
    return OArr(a.x * c, a.J * c[None], a.lap * c)


def divide(a, b):
    if _is(a) and _is(b):
        ta, tb = _bcast3(a, b)
        return OArr(*rules.div_rule(*ta, *tb))
    if _is(a):
        if isinstance(b, OConst):
            return multiply(a, OConst(1.0 / b.data))
        return multiply(a, 1.0 / np.asarray(b, dtype=a.x.dtype))
    return multiply(reciprocal(b), a)


def _as_triplet(v, like: OArr) -> OArr:
    """A constant as a triplet with zero derivatives on ``like``'s row frame."""
    if _is(v):
        return v
    d = v.data if isinstance(v, OConst) else np.asarray(v, dtype=like.x.dtype)[None]
    x = np.broadcast_to(d, np.broadcast_shapes(d.shape, like.x.shape)).astype(like.x.dtype)
    return OArr(x, np.zeros((like.J.shape[0], *x.shape), dtype=x.dtype), np.zeros_like(x))


def _binary_general(rule, a, b):
    ref = a if _is(a) else b
    ta, tb = _bcast3(_as_triplet(a, ref), _as_triplet(b, ref))
    return OArr(*rule(*ta, *tb))


def arctan2(y, x):
    return _binary_general(rules.atan2_rule, y, x)


def remainder(a, b):
    return _binary_general(rules.rem_rule, a, b)


fmod = remainder


def exp2(a):
    return exp(multiply(a, np.log(2.0)))


def split(a, indices_or_sections, axis=0):
    ax = axis % a.ndim
    n = a.shape[ax]
    cuts = [i * (n // indices_or_sections) for i in range(indices_or_sections + 1)] if np.isscalar(
        indices_or_sections) else [0, *indices_or_sections, n]
    return [getitem(a, tuple(slice(lo, hi) if d == ax else slice(None) for d in range(a.ndim)))
            for lo, hi in zip(cuts[:-1], cuts[1:])]


def stack(arrs, axis=0):
    nd = arrs[0].ndim + 1
    return concatenate([expand_dims(t, axis % nd) for t in arrs], axis=axis % nd)


def tile(a, reps):
    reps = (reps,) if np.isscalar(reps) else tuple(reps)
    nd = max(len(reps), a.ndim)
    reps = (1,) * (nd - len(reps)) + reps
    out = reshape(a, (1,) * (nd - a.ndim) + tuple(a.shape))
    for ax, r in enumerate(reps):
        if r > 1:
            out = concatenate([out] * r, axis=ax)
    return out


def dynamic_slice(a, start_indices, slice_sizes):
    idx = []
    for s0, sz, n in zip(start_indices, slice_sizes, a.shape):
        s0 = int(np.clip(int(s0), 0, n - int(sz)))
        idx.append(slice(s0, s0 + int(sz)))
    return getitem(a, tuple(idx))


def dynamic_update_slice(a, update, start_indices):
    x, J, L = a.x.copy(), a.J.copy(), a.lap.copy()
    sl = tuple(slice(int(np.clip(int(s0), 0, n - un)), int(np.clip(int(s0), 0, n - un)) + un)
               for s0, un, n in zip(start_indices, update.shape, a.shape))
    x[(slice(None), *sl)] = update.x
    J[(slice(None), slice(None), *sl)] = update.J
    L[(slice(None), *sl)] = update.lap
    return OArr(x, J, L)


def _minmax(a, b, is_max):
    if _is(a) and _is(b):
        ta, tb = _bcast3(a, b)
        return OArr(*rules.minmax_rule(*ta, *tb, is_max=is_max))
    t, c = (a, b) if _is(a) else (b, a)
    t, c = _with_const(t, c)
    shp = np.broadcast_shapes(t.x.shape, c.shape)
    cx = np.broadcast_to(c, shp)
    tx, tJ, tL = np.broadcast_to(t.x, shp), np.broadcast_to(t.J, (t.P, *shp)), np.broadcast_to(t.lap, shp)
    return OArr(*rules.minmax_rule(tx, tJ, tL, cx, np.zeros_like(tJ), np.zeros_like(tL), is_max=is_max))


def minimum(a, b):
    return _minmax(a, b, False)


def maximum(a, b):
    return _minmax(a, b, True)


def scatter(operand, idx, updates, mode='set'):
    """``operand.at[idx].set / add / min / max (updates)`` per walker with a static numpy
    index (in bounds); either argument may be a constant."""
    like = operand if _is(operand) else updates
    B, P, dt = like.B, like.P, like.x.dtype
    op_shape = tuple(operand.shape) if _is(operand) else tuple(np.shape(operand))
    S_op = int(np.prod(op_shape, dtype=int))
    tpos = np.arange(S_op).reshape(op_shape)[idx]

    def triple(v, shape):
        S = int(np.prod(shape, dtype=int))
        if _is(v):
            if tuple(v.shape) != tuple(shape):
                v = broadcast_to(v, shape)
            return v.x.reshape(B, S), v.J.reshape(v.P, B, S), v.lap.reshape(B, S)
        c = np.broadcast_to(np.asarray(v, dtype=dt), shape).reshape(1, S)
        c = np.broadcast_to(c, (B, S))
        return c, np.zeros((P, B, S), dt), np.zeros((B, S), dt)

    op3 = triple(operand, op_shape)
    up3 = triple(updates, tpos.shape)
    if op3[1].shape[0] != up3[1].shape[0]:
        Pm = max(op3[1].shape[0], up3[1].shape[0])
        ext = lambda J: np.concatenate([J, np.zeros((Pm - J.shape[0], *J.shape[1:]), J.dtype)], 0)
        op3, up3 = (op3[0], ext(op3[1]), op3[2]), (up3[0], ext(up3[1]), up3[2])
    x, J, L = rules.scatter_rule(op3, up3, tpos.reshape(-1), mode)
    return OArr(x.reshape(B, *op_shape), J.reshape(J.shape[0], B, *op_shape), L.reshape(B, *op_shape))


def _unary(name, param=None):
    def fn(a):
        if not _is(a):
            raise TypeError('oracle unary ops take triplets')
        return OArr(*rules.elementwise_rule(name, a.x, a.J, a.lap, param))

    fn.__name__ = name
    return fn


tanh = _unary('tanh')
silu = _unary('silu')
exp = _unary('exp')
log = _unary('log')
sqrt = _unary('sqrt')
rsqrt = _unary('rsqrt')
square = _unary('square')
sigmoid = _unary('logistic')
logistic = sigmoid
softplus = _unary('softplus')
sin = _unary('sin')
cos = _unary('cos')
abs = _unary('abs')
negative = _unary('neg')
log1p = _unary('log1p')
reciprocal = _unary('reciprocal')
expm1 = _unary('expm1')
sinh, cosh, tan = _unary('sinh'), _unary('cosh'), _unary('tan')
arcsin, arccos, arctan = _unary('asin'), _unary('acos'), _unary('atan')
arcsinh, arccosh, arctanh = _unary('asinh'), _unary('acosh'), _unary('atanh')
erf, erfc, erf_inv, cbrt = _unary('erf'), _unary('erfc'), _unary('erf_inv'), _unary('cbrt')
lgamma, digamma = _unary('lgamma'), _unary('digamma')


def power(a, c):
    """a ** c for a > 0: constant real exponent, or an exponent / base pair of triplets."""
    if _is(c) or isinstance(c, OConst) or not np.isscalar(c):
        return _binary_general(rules.pow_rule, a, c)
    return _unary('pow', float(c))(a)


def integer_pow(a, n):
    return OArr(*rules.elementwise_rule('integer_pow', a.x, a.J, a.lap, n))


def dot(h: OArr, W, b=None, residual=None, row_slice=None, act=None, norm=None):
    """``row_slice = (lo, hi)``: the product of ``h[..., lo:hi, :]``; ``act``: a scalar function
    applied to ``h @ W + b`` before the residual is added; ``norm = (gamma, beta, eps)``:
    ``layer_norm`` of ``h`` first."""
    if norm is not None:
        h = layer_norm(h, *norm)
    if act is not None:
        out = _unary({'sigmoid': 'logistic'}.get(act, act))(dot(h, W, b, None, row_slice))
        return out if residual is None else add(residual, out)
    if row_slice is not None:
        h = getitem(h, (Ellipsis, slice(*row_slice), slice(None)))
    W = np.asarray(W, dtype=h.x.dtype)
    bb = None if b is None else np.asarray(b, dtype=h.x.dtype)
    out = OArr(*rules.dense_rule(h.x, h.J, h.lap, W, bb))
    return out if residual is None else add(residual, out)


def exp_envelope(d, sigma, pi):
    """Exponential envelope as the chain of primitive rules the reference interprets it with."""
    e = exp(negative(multiply(expand_dims(d, -1), np.asarray(sigma))))
    return sum(multiply(e, np.asarray(pi)), axis=-2)


def layer_norm(h: OArr, gamma=None, beta=None, eps=1e-5, lazy=False):
    """LayerNorm as the chain of primitive rules the reference interprets it with (``lazy`` is
    a scheduling hint of the device front end; the value is the same)."""
    mu = mean(h, axis=-1, keepdims=True)
    c = subtract(h, mu)
    var = mean(square(c), axis=-1, keepdims=True)
    y = multiply(c, rsqrt(add(var, eps)))
    if gamma is not None:
        y = multiply(y, gamma)
    return y if beta is None else add(y, beta)


def sum(a: OArr, axis=None, keepdims=False, window=None):
    """``window = (lo, hi)``: the sum of the slice ``lo:hi`` along the (single) axis."""
    if axis is None:
        axis = tuple(range(a.ndim))
    if window is not None:
        ax = int(np.atleast_1d(axis)[0]) % a.ndim
        a = getitem(a, tuple(slice(*window) if i == ax else slice(None) for i in range(ax + 1)))
    return OArr(*rules.sum_rule(a.x, a.J, a.lap, axis, keepdims))


def mean(a: OArr, axis=None, keepdims=False, window=None):
    if axis is None:
        axis = tuple(range(a.ndim))
    n = int(np.prod([a.shape[i] for i in np.atleast_1d(axis)])) if window is None else int(window[1] - window[0])
    return multiply(sum(a, axis, keepdims, window), 1.0 / n)


def reshape(a: OArr, shape):
    shape = tuple(shape)
    return OArr(
        a.x.reshape(a.B, *shape), a.J.reshape(a.P, a.B, *shape), a.lap.reshape(a.B, *shape)
    )


def transpose(a: OArr, axes):
    axes = tuple(ax % a.ndim for ax in axes)
    xa = (0, *[ax + 1 for ax in axes])
    ja = (0, 1, *[ax + 2 for ax in axes])
    return OArr(a.x.transpose(xa), a.J.transpose(ja), a.lap.transpose(xa))


def swapaxes(a: OArr, i, j):
    axes = list(range(a.ndim))
    axes[i], axes[j] = axes[j], axes[i]
    return transpose(a, axes)


def expand_dims(a: OArr, axis):
    axis = axis % (a.ndim + 1)
    return OArr(
        np.expand_dims(a.x, axis + 1), np.expand_dims(a.J, axis + 2), np.expand_dims(a.lap, axis + 1)
    )


def broadcast_to(a: OArr, shape, lazy=False):
    shape = tuple(shape)  # ``lazy`` is a scheduling hint of the device front end; the value is the same
    ex = len(shape) - a.ndim
    x = a.x.reshape(a.B, *([1] * ex), *a.shape)
    J = a.J.reshape(a.P, a.B, *([1] * ex), *a.shape)
    L = a.lap.reshape(a.B, *([1] * ex), *a.shape)
    return OArr(
        np.broadcast_to(x, (a.B, *shape)).copy(),
        np.broadcast_to(J, (a.P, a.B, *shape)).copy(),
        np.broadcast_to(L, (a.B, *shape)).copy(),
    )


def getitem(a: OArr, idx):
    if not isinstance(idx, tuple):
        idx = (idx,)
    return OArr(
        a.x[(slice(None), *idx)], a.J[(slice(None), slice(None), *idx)], a.lap[(slice(None), *idx)]
    )


def concatenate(arrs, axis=-1, lazy=False):
    first = [t for t in arrs if _is(t)][0]
    nd = first.ndim
    axis = axis % nd
    P = max(t.P for t in arrs if _is(t))
    xs, Js, Ls = [], [], []
    for t in arrs:
        if _is(t):
            J = t.J
            if J.shape[0] < P:
                J = np.concatenate([J, np.zeros((P - J.shape[0], *J.shape[1:]), J.dtype)], 0)
            xs.append(t.x), Js.append(J), Ls.append(t.lap)
        else:
            c = np.asarray(t, dtype=first.x.dtype)
            c = np.broadcast_to(c[None], (first.B, *c.shape))
            xs.append(c)
            Js.append(np.zeros((P, *c.shape), c.dtype))
            Ls.append(np.zeros_like(c))
    return OArr(
        np.concatenate(xs, axis + 1), np.concatenate(Js, axis + 2), np.concatenate(Ls, axis + 1)
    )


def stop_gradient(a):
    return OConst(a.x) if _is(a) else a


def amax_const(a, axis, keepdims=False):
    """max over ``axis`` of the values only, as a walker-varying constant."""
    x = a.x if _is(a) else a.data
    ax = tuple(i % (x.ndim - 1) + 1 for i in np.atleast_1d(axis))
    return OConst(x.max(ax, keepdims=keepdims))


def sign(a):
    return OConst(np.sign(a.x if _is(a) else a.data))


def squeeze(a: OArr, axis):
    shape = list(a.shape)
    del shape[axis % a.ndim]
    return reshape(a, shape)


def logsumexp(a: OArr, axis=-1, b=None):
    """Same primitive sequence as ``jax.nn.logsumexp(..., b=b, return_sign=True)``."""
    m = amax_const(a, axis, keepdims=True)
    e = exp(subtract(a, m))
    if b is not None:
        e = multiply(e, b)
    s = sum(e, axis)
    val = add(log(abs(s)), OConst(m.data.reshape(s.x.shape)))
    return val, sign(s)


def _letters(n, used=''):
    pool = [c for c in 'abcdefghijklmnopqrstuvwx' if c not in used]
    return ''.join(pool[:n])


def dot_general(lhs, rhs, dimension_numbers):
    """``jax.lax.dot_general`` on triplets and constants (output axes: batch, lhs free, rhs free),
    evaluated as one einsum (folx/wrapped_functions.py:71-171 for one constant operand,
    :174-309 for two operands with derivatives)."""
    (lc, rc), (lb, rb) = dimension_numbers
    nl, nr = len(np.shape(lhs) if not _is(lhs) else lhs.shape), len(np.shape(rhs) if not _is(rhs) else rhs.shape)
    lc, lb = [i % nl for i in lc], [i % nl for i in lb]
    rc, rb = [i % nr for i in rc], [i % nr for i in rb]
    sl = list(_letters(nl))
    sr = list(_letters(nr, used=''.join(sl)))
    for i, j in zip(lc, rc):
        sr[j] = sl[i]
    for i, j in zip(lb, rb):
        sr[j] = sl[i]
    out = [sl[i] for i in lb] + [c for i, c in enumerate(sl) if i not in lc and i not in lb] \
        + [c for j, c in enumerate(sr) if j not in rc and j not in rb]
    sub = f"{''.join(sl)},{''.join(sr)}->{''.join(out)}"
    if not _is(lhs) and not _is(rhs):
        return np.einsum(sub, np.asarray(lhs), np.asarray(rhs))
    return einsum(sub, lhs, rhs)


def matmul(a, b):
    """numpy.matmul semantics (1-D operands are vectors, leading axes broadcast); either operand may
    be a constant of any rank.  Two triplets with equal leading axes go through
    ``rules.dot_two_rule`` (the dot_last path of the reference, folx/wrapped_functions.py:294-309);
    everything else is the same contraction written as an einsum."""
    if _is(a) and _is(b) and a.shape[:-2] == b.shape[:-2] and a.ndim >= 2 and b.ndim >= 2:
        Ja, Jb = _padJ(a, b)
        return OArr(*rules.dot_two_rule(a.x, Ja, a.lap, b.x, Jb, b.lap))
    sa = tuple(a.shape) if _is(a) else np.shape(a)
    sb = tuple(b.shape) if _is(b) else np.shape(b)
    av, bv = len(sa) == 1, len(sb) == 1
    la, lb = ([] if av else list(sa[:-2])), ([] if bv else list(sb[:-2]))
    L = max(len(la), len(lb))
    lead = _letters(L)
    # numpy's einsum broadcasts axes of size 1 that share a letter with a longer axis, as matmul does
    sa_ = lead[L - len(la):] + ('' if av else 'y') + 'z'
    sb_ = lead[L - len(lb):] + 'z' + ('' if bv else 'w')
    out = lead + ('' if av else 'y') + ('' if bv else 'w')
    return einsum(f'{sa_},{sb_}->{out}', a, b)


def _einsum_terms(subscripts, ranks):
    """Ellipsis and implicit-output forms of numpy.einsum written out with explicit letters."""
    spec = subscripts.replace(' ', '')
    ins, arrow, out = spec.partition('->')
    terms = ins.split(',')
    n_ell = [r - (len(t) - 3) if '...' in t else 0 for t, r in zip(terms, ranks)]
    width = max(n_ell) if n_ell else 0
    ell = ''.join([c for c in 'ABCDEFGHIJKLMNOPQRSTUVWX' if c not in spec][:width])
    terms = [t.replace('...', ell[width - n:] if n else '') for t, n in zip(terms, n_ell)]
    if arrow:
        out = out.replace('...', ell)
    else:
        joined = ''.join(terms)
        out = ell + ''.join(sorted(c for c in set(joined) if joined.count(c) == 1 and c not in ell))
    return terms, out


def einsum(subscripts, *ops):
    """einsum of any number of triplets and constants, evaluated directly: the function is linear in every operand,
    so J = sum_k f(.., J_k, ..), lap = sum_k f(.., lap_k, ..) + 2 sum_{k<l} sum_p f(.., J_k,p, .., J_l,p, ..)
    (folx/hessian.py:177-188 for two operands)."""
    terms, out = _einsum_terms(subscripts, [o.ndim if _is(o) else np.ndim(o) for o in ops])
    trip = [k for k, o in enumerate(ops) if _is(o)]
    assert trip, 'einsum: no triplet among the operands'
    P = max(ops[k].P for k in trip)
    padJ = {k: np.concatenate([ops[k].J, np.zeros((P - ops[k].P, *ops[k].J.shape[1:]), ops[k].J.dtype)], 0) for k in trip}

    def ev(subst, lead_out):          # subst: {operand index: (array, leading letters)}; the others contribute their value
        arrs, subs = [], []
        for k, (o, t) in enumerate(zip(ops, terms)):
            if k in subst:
                arr, lead = subst[k]
            elif _is(o):
                arr, lead = o.x, 'Z'
            else:
                arr, lead = np.asarray(o), ''
            arrs.append(arr)
            subs.append(lead + t)
        return np.einsum(','.join(subs) + '->' + lead_out + out, *arrs)

    x = ev({}, 'Z')
    J = builtins_sum(ev({k: (padJ[k], 'YZ')}, 'YZ') for k in trip)
    lap = builtins_sum(ev({k: (ops[k].lap, 'Z')}, 'Z') for k in trip)
    for a_, k in enumerate(trip):
        for l in trip[a_ + 1:]:
            lap = lap + 2.0 * ev({k: (padJ[k], 'YZ'), l: (padJ[l], 'YZ')}, 'Z')
    return OArr(x, J, lap)


def softmax(a: OArr, axis=-1):
    e = exp(subtract(a, amax_const(a, axis, keepdims=True)))
    return divide(e, sum(e, axis, keepdims=True))


def det(A: OArr):
    """det = sign * exp(logdet) (folx/slogdet.py:361-395)."""
    sg, ld = slogdet(A)
    return multiply(exp(ld), sg)


def slogdet(A: OArr, row_axis=None, factor=None):
    if factor is not None:
        A = multiply(A, factor)
    if row_axis is not None and row_axis % A.ndim != A.ndim - 2:
        perm = [a for a in range(A.ndim) if a != row_axis % A.ndim]
        perm.insert(A.ndim - 2, row_axis % A.ndim)
        A = transpose(A, perm)
    sign, (ld, J, L) = rules.slogdet_rule(A.x, A.J, A.lap)
    return OConst(sign), OArr(ld, J, L)


def inv(A: OArr):
    """Matrix inverse (folx/linear_solve.py:114-145)."""
    return OArr(*rules.inv_rule(A.x, A.J, A.lap))


def solve(A, b):
    """``numpy.linalg.solve`` semantics per walker (folx/linear_solve.py:54-111): ``b`` of
    logical rank 1 is a vector, anything else a stack of matrices; batch axes broadcast
    from the right, the solution carries the broadcast batch shape.  Either operand may
    be a constant."""
    like = A if _is(A) else b
    assert _is(like), 'solve of two constants is not a forward-Laplacian rule'
    B = like.B

    def parts(v, tail):
        # -> x (B|1, *batch, *tail axes), J or None, lap or None, logical batch ndim
        if _is(v):
            return v.x, v.J, v.lap
        c, _ = _const(v, like)
        return c, None, None

    Ax, AJ, AL = parts(A, 2)
    bx, bJ, bL = parts(b, None)
    vector = bx.ndim - 1 == 1
    if vector:
        bx = bx[..., None]
        bJ = None if bJ is None else bJ[..., None]
        bL = None if bL is None else bL[..., None]
    nb = max(Ax.ndim - 3, bx.ndim - 3)  # logical batch axes of the solution

    def lift(x, lead):
        # insert missing batch axes right behind the leading ``lead`` axes
        if x is None:
            return None
        missing = nb - (x.ndim - lead - 2)
        return x.reshape(*x.shape[:lead], *([1] * missing), *x.shape[lead:])

    Ax, AL, bx, bL = lift(Ax, 1), lift(AL, 1), lift(bx, 1), lift(bL, 1)
    AJ, bJ = lift(AJ, 2), lift(bJ, 2)
    batch = np.broadcast_shapes(Ax.shape[1:-2], bx.shape[1:-2])
    n, m = bx.shape[-2:]
    full_A, full_b = (B, *batch, n, n), (B, *batch, n, m)
    if AJ is not None and bJ is not None and AJ.shape[0] != bJ.shape[0]:
        P = max(AJ.shape[0], bJ.shape[0])
        AJ = np.concatenate([AJ, np.zeros((P - AJ.shape[0], *AJ.shape[1:]), AJ.dtype)], 0)
        bJ = np.concatenate([bJ, np.zeros((P - bJ.shape[0], *bJ.shape[1:]), bJ.dtype)], 0)
    bc = lambda x, shape: None if x is None else np.broadcast_to(x, shape)
    P = (AJ if AJ is not None else bJ).shape[0]
    y, yJ, yL = rules.solve_rule(bc(Ax, full_A), bc(AJ, (P, *full_A)), bc(AL, full_A),
                                 bc(bx, full_b), bc(bJ, (P, *full_b)), bc(bL, full_b))
    if vector:
        y, yJ, yL = y[..., 0], yJ[..., 0], yL[..., 0]
    return OArr(y, yJ, yL)


def multi_head_self_attention(q: OArr, k: OArr, v: OArr, mask=None, input_mask=None, bias=None):
    """``bias`` = optional edge-bias triplet of per-walker shape (n, H, n)."""
    if bias is None:
        o, oJ, oL = rules.mhsa_rule(q.x, q.J, q.lap, k.x, k.J, k.lap, v.x, v.J, v.lap, mask, input_mask)
    else:
        o, oJ, oL = rules.mhsa_rule(q.x, q.J, q.lap, k.x, k.J, k.lap, v.x, v.J, v.lap, mask, input_mask,
                                    bias.x, bias.J, bias.lap)
    return OArr(o, oJ, oL)


def to_numpy(a):
    return a


def clip(a: OArr, lo=None, hi=None):
    """Constant bounds: inside the bounds the triplet passes, outside it is constant."""
    lo_ = -np.inf if lo is None else lo
    hi_ = np.inf if hi is None else hi
    inside = ((a.x > lo_) & (a.x < hi_)).astype(a.x.dtype)
    edge = 0.5 * ((a.x == lo_) | (a.x == hi_))  # jax splits a tie between the two arguments
    w = inside + edge
    return OArr(np.clip(a.x, lo_, hi_), a.J * w[None], a.lap * w)


def where(cond, a, b):
    """``numpy.where`` with numpy's broadcasting over the PER-SAMPLE shapes (operands of lower rank are aligned on the
    right, behind the walker axis)."""
    c = np.asarray(cond.data if isinstance(cond, OConst) else cond).astype(bool)
    per_walker_cond = isinstance(cond, OConst)
    like = a if _is(a) else b
    B, dt = like.x.shape[0], like.x.dtype
    shapes = [c.shape[1:] if per_walker_cond else c.shape] + [v.x.shape[1:] if _is(v) else np.shape(v) for v in (a, b)]
    full = np.broadcast_shapes(*shapes)
    nd = len(full)

    def lift(t, lead):      # t has `lead` leading axes (rows, walkers) in front of its per-sample shape
        t = t.reshape((*t.shape[:lead], *((1,) * (nd - (t.ndim - lead))), *t.shape[lead:]))
        return np.broadcast_to(t, (*t.shape[:lead], *full))

    c = lift(c, 1) if per_walker_cond else np.broadcast_to(lift(c, 0)[None], (B, *full))
    P = max([v.J.shape[0] for v in (a, b) if _is(v)])

    def trip(v):
        if _is(v):
            J = np.concatenate([v.J, np.zeros((P - v.J.shape[0], *v.J.shape[1:]), v.J.dtype)], 0)
            return lift(v.x, 1), lift(J, 2), lift(v.lap, 1)
        cv = np.broadcast_to(lift(np.asarray(v, dtype=dt), 0)[None], (B, *full))
        return cv, np.zeros((P, B, *full), dt), np.zeros((B, *full), dt)

    (ax, aJ, aL), (bx, bJ, bL) = trip(a), trip(b)
    return OArr(np.where(c, ax, bx), np.where(c[None], aJ, bJ), np.where(c, aL, bL))


def cumsum(a: OArr, axis=-1):
    ax = axis % a.ndim
    return OArr(np.cumsum(a.x, ax + 1), np.cumsum(a.J, ax + 2), np.cumsum(a.lap, ax + 1))


def _arg_reduce(a: OArr, axis, fn):
    ax = axis % a.ndim
    idx = np.expand_dims(fn(a.x, axis=ax + 1), ax + 1)
    tk = lambda t, off: np.squeeze(np.take_along_axis(t, idx if off == 1 else idx[None].repeat(t.shape[0], 0),
                                                      ax + off), ax + off)
    return OArr(tk(a.x, 1), tk(a.J, 2), tk(a.lap, 1))


def amax(a: OArr, axis=-1):
    return _arg_reduce(a, axis, np.argmax)


def amin(a: OArr, axis=-1):
    return _arg_reduce(a, axis, np.argmin)


def prod(a: OArr, axis=-1):
    """f = prod x_i (all x_i != 0): grad_i = f / x_i, H_ij = f / (x_i x_j) for i != j."""
    ax = axis % a.ndim
    f = np.prod(a.x, ax + 1)
    g = np.expand_dims(f, ax + 1) / a.x                       # f / x_i
    J = (np.expand_dims(g, 0) * a.J).sum(ax + 2)
    r = a.J / a.x[None]                                        # J_pi / x_i
    cross = (r.sum(ax + 2) ** 2 - (r * r).sum(ax + 2)).sum(0)  # sum_p sum_{i != j} r_pi r_pj
    return OArr(f, J, (g * a.lap).sum(ax + 1) + f * cross)


def flip(a: OArr, axis):
    axes = (axis,) if np.isscalar(axis) else tuple(axis)
    ax = tuple(x % a.ndim for x in axes)
    return OArr(np.flip(a.x, tuple(x + 1 for x in ax)), np.flip(a.J, tuple(x + 2 for x in ax)),
                np.flip(a.lap, tuple(x + 1 for x in ax)))


def pad(a: OArr, pad_width, constant_values=0.0):
    pw = [tuple(p) for p in pad_width] if np.ndim(pad_width) == 2 else [tuple(pad_width)] * a.ndim
    return OArr(np.pad(a.x, [(0, 0)] + pw, constant_values=constant_values), np.pad(a.J, [(0, 0), (0, 0)] + pw),
                np.pad(a.lap, [(0, 0)] + pw))


def lax_pad(a: OArr, padding_value, padding_config):
    """``jax.lax.pad`` semantics (what folx wraps as an indexing rule, folx/wrapped_functions.py:480-487), written
    as array surgery: a canvas of the padding value, the operand laid out with strides ``interior + 1``, then the
    low / high edges added or (negative) cut.  The padding value may carry derivatives."""
    cfg = [tuple(int(v) for v in c) for c in padding_config]

    def one(arr, lead, fill):          # arr (*lead_shape, *shape); fill broadcastable to lead_shape
        shape = arr.shape[lead:]
        dil = [n + max(n - 1, 0) * it for n, (_, _, it) in zip(shape, cfg)]
        canvas = np.empty((*arr.shape[:lead], *dil), dtype=arr.dtype)
        canvas[...] = np.asarray(fill).reshape(*np.shape(fill), *([1] * len(shape)))
        canvas[(*[slice(None)] * lead, *[slice(None, None, it + 1) for (_, _, it) in cfg])] = arr
        for ax, (lo, hi, _) in enumerate(cfg):
            n = canvas.shape[lead + ax]
            canvas = canvas[(*[slice(None)] * (lead + ax), slice(max(-lo, 0), n - max(-hi, 0)))]
            edge = lambda w: np.broadcast_to(
                np.asarray(fill).reshape(*np.shape(fill), *([1] * len(shape))),
                (*canvas.shape[:lead + ax], w, *canvas.shape[lead + ax + 1:]))
            canvas = np.concatenate([edge(max(lo, 0)), canvas, edge(max(hi, 0))], axis=lead + ax)
        return canvas

    B, P = a.x.shape[0], a.J.shape[0]
    if _is(padding_value):
        fx, fJ, fl = padding_value.x.reshape(B), padding_value.J.reshape(P, B), padding_value.lap.reshape(B)
    else:
        fx, fJ, fl = np.full(B, float(np.asarray(padding_value))), np.zeros((P, B)), np.zeros(B)
    return OArr(one(a.x, 1, fx), one(a.J, 2, fJ), one(a.lap, 1, fl))


def _cmp(fn):
    def f(a, b):
        av = a.x if _is(a) else np.asarray(a)
        bv = b.x if _is(b) else np.asarray(b)
        return OConst(fn(av, bv))

    return f


greater, greater_equal, less, less_equal = _cmp(np.greater), _cmp(np.greater_equal), _cmp(np.less), _cmp(np.less_equal)


def floor(a):
    return OConst(np.floor(a.x))


def logaddexp(a: OArr, b: OArr):
    """From the Hessian of log(e^a + e^b): weights s = sigmoid(a - b), curvature s (1 - s)."""
    (ax, aJ, aL), (bx, bJ, bL) = _bcast3(a, b)
    s = 1.0 / (1.0 + np.exp(bx - ax))
    d = aJ - bJ
    return OArr(np.logaddexp(ax, bx), s * aJ + (1 - s) * bJ, s * aL + (1 - s) * bL + s * (1 - s) * (d * d).sum(0))


def cumprod(a: OArr, axis=-1):
    ax = axis % a.ndim
    n = a.shape[ax]
    parts = [prod(getitem(a, tuple(slice(0, i + 1) if d == ax else slice(None) for d in range(a.ndim))), axis=ax)
             for i in range(n)]
    return OArr(np.stack([p.x for p in parts], ax + 1), np.stack([p.J for p in parts], ax + 2),
                np.stack([p.lap for p in parts], ax + 1))


def _cumarg(a: OArr, axis, red):
    ax = axis % a.ndim
    n = a.shape[ax]
    parts = [red(getitem(a, tuple(slice(0, i + 1) if d == ax else slice(None) for d in range(a.ndim))), axis=ax)
             for i in range(n)]
    return OArr(np.stack([p.x for p in parts], ax + 1), np.stack([p.J for p in parts], ax + 2),
                np.stack([p.lap for p in parts], ax + 1))


def cummax(a: OArr, axis=-1):
    return _cumarg(a, axis, amax)


def cummin(a: OArr, axis=-1):
    return _cumarg(a, axis, amin)


# jax.numpy / jax.nn names that the reference traces into chains of primitives -----------------------
def _fields(a: OArr, fn):
    """The same array surgery on the three fields; ``fn(t, lead)`` sees ``lead`` leading non-logical axes."""
    return OArr(fn(a.x, 1), fn(a.J, 2), fn(a.lap, 1))


def relu(a):
    return maximum(a, 0.0)


def leaky_relu(a, negative_slope=0.01):
    return where(greater_equal(a, 0.0), a, multiply(a, float(negative_slope)))


def elu(a, alpha=1.0):
    return where(greater(a, 0.0), a, multiply(expm1(minimum(a, 0.0)), float(alpha)))


def gelu(a, approximate=True):
    if approximate:
        u = multiply(add(a, multiply(integer_pow(a, 3), 0.044715)), float(np.sqrt(2.0 / np.pi)))
        return multiply(multiply(a, 0.5), add(tanh(u), 1.0))
    return multiply(multiply(a, 0.5), add(erf(multiply(a, float(1.0 / np.sqrt(2.0)))), 1.0))


def log_softmax(a, axis=-1):
    val, _ = logsumexp(a, axis)
    return subtract(a, expand_dims(val, axis))


def var(a, axis=None, keepdims=False):
    m2 = mean(square(a), axis, keepdims)
    return subtract(m2, square(mean(a, axis, keepdims)))


def std(a, axis=None, keepdims=False):
    return sqrt(var(a, axis, keepdims))


def norm(a, axis=None, keepdims=False):
    return sqrt(sum(square(a), axis, keepdims))


def vdot(a, b):
    return sum(multiply(reshape(a, (-1,)) if _is(a) else np.reshape(a, -1), reshape(b, (-1,)) if _is(b) else np.reshape(b, -1)))


def tensordot(a, b, axes=2):
    nda = a.ndim if _is(a) else np.ndim(a)
    ndb = b.ndim if _is(b) else np.ndim(b)
    if isinstance(axes, int):
        ca, cb = tuple(range(nda - axes, nda)), tuple(range(axes))
    else:
        ca, cb = [(v,) if isinstance(v, int) else tuple(v) for v in axes]
    return dot_general(a, b, ((tuple(i % nda for i in ca), tuple(i % ndb for i in cb)), ((), ())))


def inner(a, b):
    return tensordot(a, b, axes=((-1,), (-1,)))


def outer(a, b):
    return multiply(reshape(a, (-1, 1)), reshape(b, (1, -1)))


def moveaxis(a: OArr, source, destination):
    src = (source,) if isinstance(source, int) else tuple(source)
    dst = (destination,) if isinstance(destination, int) else tuple(destination)
    return _fields(a, lambda t, lead: np.moveaxis(t, [s % a.ndim + lead for s in src], [d % a.ndim + lead for d in dst]))


def take(a: OArr, indices, axis=None):
    idx = np.asarray(indices)
    if axis is None:
        return _fields(reshape(a, (-1,)), lambda t, lead: np.take(t, idx, axis=lead))
    return _fields(a, lambda t, lead: np.take(t, idx, axis=axis % a.ndim + lead))


def diagonal(a: OArr, offset=0):
    return _fields(a, lambda t, lead: np.diagonal(t, offset, -2, -1))


def trace(a: OArr, offset=0):
    return _fields(a, lambda t, lead: np.trace(t, offset, -2, -1))


def roll(a: OArr, shift, axis):
    return _fields(a, lambda t, lead: np.roll(t, shift, axis % a.ndim + lead))


def repeat(a: OArr, repeats, axis):
    return _fields(a, lambda t, lead: np.repeat(t, repeats, axis % a.ndim + lead))

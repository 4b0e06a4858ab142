"""Numpy restatement of the forward-Laplacian propagation rules (test infrastructure).

Every rule maps input triplets ``(x, J, lap)`` to the output triplet following

    y     = f(x)
    J_y   = J_f . J                              (folx/jvp.py:676-711)
    lap_y = J_f . lap + tr(J^T H_f J)            (folx/wrapper.py:120-125)

Arrays use the layout ``x (B, *s)``, ``J (P, B, *s)``, ``lap (B, *s)``.  All functions
work in the dtype of their inputs (float64 for pinning, float32 for the CPU baseline).
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------------------
# Elementwise activations: (f, f', f'') in closed form.
# Reference: f'(x) comes from a vjp with ones (folx/jvp.py:687-697, :262-272), f''(x)
# from jvp-of-jvp (folx/hessian.py:87-112); the closed forms below are what those AD
# calls evaluate to for each registered primitive (folx/wrapped_functions.py:385-415,
# :552-560, :622-625).
# --------------------------------------------------------------------------------------


def _sigmoid(x):
    # numerically stable logistic
    out = np.empty_like(x)
    pos = x >= 0
    out[pos] = 1.0 / (1.0 + np.exp(-x[pos]))
    e = np.exp(x[~pos])
    out[~pos] = e / (1.0 + e)
    return out


def _tanh(x):
    t = np.tanh(x)
    return t, 1 - t * t, -2 * t * (1 - t * t)


def _silu(x):
    s = _sigmoid(x)
    return x * s, s * (1 + x * (1 - s)), s * (1 - s) * (2 + x * (1 - 2 * s))


def _exp(x):
    e = np.exp(x)
    return e, e, e


def _log(x):
    return np.log(x), 1 / x, -1 / (x * x)


def _sqrt(x):
    r = np.sqrt(x)
    return r, 0.5 / r, -0.25 / (r * x)


def _rsqrt(x):
    r = 1 / np.sqrt(x)
    return r, -0.5 * r / x, 0.75 * r / (x * x)


def _square(x):
    return x * x, 2 * x, np.full_like(x, 2.0)


def _logistic(x):
    s = _sigmoid(x)
    return s, s * (1 - s), s * (1 - s) * (1 - 2 * s)


def _softplus(x):
    s = _sigmoid(x)
    return np.logaddexp(x, 0), s, s * (1 - s)


def _sin(x):
    return np.sin(x), np.cos(x), -np.sin(x)


def _cos(x):
    return np.cos(x), -np.sin(x), -np.cos(x)


def _abs(x):
    # registered LINEAR (folx/wrapped_functions.py:349-352): no Hessian term
    return np.abs(x), np.sign(x), np.zeros_like(x)


def _neg(x):
    return -x, np.full_like(x, -1.0), np.zeros_like(x)


def _log1p(x):
    return np.log1p(x), 1 / (1 + x), -1 / ((1 + x) * (1 + x))


def _reciprocal(x):
    r = 1 / x
    return r, -r * r, 2 * r * r * r


def _expm1(x):
    e = np.exp(x)
    return np.expm1(x), e, e


def _sinh(x):
    return np.sinh(x), np.cosh(x), np.sinh(x)


def _cosh(x):
    return np.cosh(x), np.sinh(x), np.cosh(x)


def _tan(x):
    t = np.tan(x)
    return t, 1 + t * t, 2 * t * (1 + t * t)


def _asin(x):
    r = 1 / np.sqrt(1 - x * x)
    return np.arcsin(x), r, x * r**3


def _acos(x):
    r = 1 / np.sqrt(1 - x * x)
    return np.arccos(x), -r, -x * r**3


def _atan(x):
    q = 1 / (1 + x * x)
    return np.arctan(x), q, -2 * x * q * q


def _asinh(x):
    r = 1 / np.sqrt(1 + x * x)
    return np.arcsinh(x), r, -x * r**3


def _acosh(x):
    r = 1 / np.sqrt(x * x - 1)
    return np.arccosh(x), r, -x * r**3


def _atanh(x):
    q = 1 / (1 - x * x)
    return np.arctanh(x), q, 2 * x * q * q


def _erf(x):
    from scipy.special import erf

    g = 2 / np.sqrt(np.pi) * np.exp(-x * x)
    return erf(x), g, -2 * x * g


def _erfc(x):
    from scipy.special import erfc

    g = 2 / np.sqrt(np.pi) * np.exp(-x * x)
    return erfc(x), -g, 2 * x * g


def _erf_inv(x):
    from scipy.special import erfinv

    v = erfinv(x)
    g = np.sqrt(np.pi) / 2 * np.exp(v * v)
    return v, g, 2 * v * g * g


def _cbrt(x):
    c = np.cbrt(x)
    return c, c / (3 * x), -2 * c / (9 * x * x)


def _lgamma(x):
    from scipy.special import digamma, gammaln, polygamma

    return gammaln(x), digamma(x), polygamma(1, x)


def _digamma(x):
    """Values from scipy for x > 0 (its polygamma is defined there); negative arguments by the
    reflection formulas psi1(1-x) + psi1(x) = pi^2 / sin^2(pi x) and
    psi2(1-x) - psi2(x) = 2 pi^3 cos(pi x) / sin^3(pi x)."""
    from scipy.special import digamma, polygamma

    xp = np.where(x > 0, x, 1 - x)
    p1, p2 = polygamma(1, xp), polygamma(2, xp)
    s, c = np.sin(np.pi * x), np.cos(np.pi * x)
    p1 = np.where(x > 0, p1, np.pi ** 2 / s ** 2 - p1)
    p2 = np.where(x > 0, p2, p2 - 2 * np.pi ** 3 * c / s ** 3)
    return digamma(x), p1, p2


def _identity(x):
    return x, np.ones_like(x), np.zeros_like(x)


ACTIVATIONS = {
    'tanh': _tanh,
    'silu': _silu,
    'exp': _exp,
    'log': _log,
    'sqrt': _sqrt,
    'rsqrt': _rsqrt,
    'square': _square,
    'logistic': _logistic,
    'sigmoid': _logistic,
    'softplus': _softplus,
    'sin': _sin,
    'cos': _cos,
    'abs': _abs,
    'neg': _neg,
    'log1p': _log1p,
    'reciprocal': _reciprocal,
    'expm1': _expm1,
    'identity': _identity,
    # the rest of the reference's scalar table (folx/wrapped_functions.py:416-445)
    'sinh': _sinh, 'cosh': _cosh, 'tan': _tan, 'asin': _asin, 'acos': _acos, 'atan': _atan,
    'asinh': _asinh, 'acosh': _acosh, 'atanh': _atanh, 'erf': _erf, 'erfc': _erfc, 'erf_inv': _erf_inv,
    'cbrt': _cbrt, 'lgamma': _lgamma, 'digamma': _digamma,
}


def integer_pow(x, n: int):
    """``lax.integer_pow`` closed forms (folx/wrapped_functions.py:385)."""
    return x**n, n * x ** (n - 1), n * (n - 1) * x ** (n - 2)


def elementwise_rule(name, x, J, lap, param=None):
    """y = f(x); J_y = f'(x) * J; lap_y = f'(x) * lap + f''(x) * sum_p J_p^2.

    folx/jvp.py:687-697 (dense), folx/jvp.py:262-272 (sparse rows, mask unchanged),
    folx/hessian.py:87-112 (sum over the Jacobian axis of J*J, valid for sparse storage
    when no index repeats per position), combined at folx/wrapper.py:120-125.
    """
    if name == 'integer_pow':
        y, d1, d2 = integer_pow(x, int(param))
    elif name == 'pow':  # x^param, x > 0, constant real exponent (jax.lax.pow_p)
        y, d1, d2 = x**param, param * x ** (param - 1), param * (param - 1) * x ** (param - 2)
    elif name == 'scale':  # y = param * x, linear
        y, d1, d2 = param * x, np.full_like(x, param), np.zeros_like(x)
    else:
        y, d1, d2 = ACTIVATIONS[name](x)
    Jy = d1[None] * J
    lapy = d1 * lap + d2 * (J * J).sum(0)
    return y, Jy, lapy


# --------------------------------------------------------------------------------------
# Dense layer: one operand carries derivatives, the other is constant.
# --------------------------------------------------------------------------------------


def dense_rule(x, J, lap, W, b=None):
    """y = x @ W (+ b) along the last axis; the op is linear so the same product is
    applied to x, to every Jacobian row and to the Laplacian
    (folx/wrapped_functions.py:167-169).  A constant bias shifts x only
    (``add`` is LINEAR, folx/wrapped_functions.py:365-367)."""
    y = x @ W
    if b is not None:
        y = y + b
    return y, J @ W, lap @ W


def dot_const_rule(a, Ja, La, W):
    """y = a @ W over the last two axes, ``a (.., Bt, I, Kc)`` with derivatives and ``W (Bt, Kc, J)`` a
    constant with a batch axis (per-head weights): ``_dot_general_one_constant`` with batch
    dimensions on the constant (folx/wrapped_functions.py:71-171); the product is linear in ``a``,
    so it is applied to x, to every Jacobian row and to the Laplacian (:167-169).
    Pinned by AD Hessian traces of per-head products in tests/test_oracle_rules.py."""
    return a @ W, Ja @ W, La @ W


def dot_two_rule(a, Ja, La, b, Jb, Lb):
    """y = a @ b over the last two axes with BOTH operands carrying derivatives (dense Jacobians
    on the same rows): the product is linear in each operand (JVP both ways,
    folx/jvp.py:676-684) and its Hessian couples the two operands through the identity, so
    tr(J^T H J) = 2 sum_p Ja_p @ Jb_p (dot_product_jac_hessian_jac, folx/hessian.py:177-188,
    for the dot_last einsum of folx/wrapped_functions.py:294-309).
    Pinned by AD Hessian traces in tests/test_oracle_rules.py and by equality with the
    multiply-and-sum decomposition (mul_rule + sum_rule)."""
    y = a @ b
    Jy = Ja @ b[None] + a[None] @ Jb
    lap = La @ b + a @ Lb + 2.0 * np.einsum('p...ik,p...kj->...ij', Ja, Jb)
    return y, Jy, lap


# --------------------------------------------------------------------------------------
# Binary elementwise rules with both operands carrying derivatives (dense Jacobians).
# --------------------------------------------------------------------------------------


def _bc(*arrs):
    return np.broadcast_arrays(*arrs)


def mul_rule(a, Ja, La, b, Jb, Lb):
    """y = a * b.  JVP by linearity in each argument (folx/jvp.py:676-684); the Hessian
    is the off-diagonal identity so tr(J^T H J) = 2 sum_p Ja_p * Jb_p
    (folx/hessian.py:177-188, MULTIPLICATION flag folx/wrapped_functions.py:377-379)."""
    y = a * b
    Jy = a[None] * Jb + b[None] * Ja
    lap = a * Lb + b * La + 2 * (Ja * Jb).sum(0)
    return y, Jy, lap


def div_rule(a, Ja, La, b, Jb, Lb):
    """y = a / b with the custom Hessian of folx/custom_hessian.py:35-59:
    H_lr = -2 / b^2 (counted once for the symmetric pair), H_rr = 2 a / b^3."""
    y = a / b
    rb2 = 1 / (b * b)
    Jy = Ja / b[None] - (a * rb2)[None] * Jb
    lap = La / b - a * rb2 * Lb
    lap = lap + (-2 * rb2) * (Ja * Jb).sum(0) + (2 * a * rb2 / b) * (Jb * Jb).sum(0)
    return y, Jy, lap


def binary_hessian_rule(y, fa, fb, faa, fab, fbb, Ja, La, Jb, Lb):
    """General two-argument scalar function from its value, gradient (fa, fb) and Hessian
    (faa, fab, fbb) at every element -- what ``wrap_forward_laplacian`` of a binary jax
    function evaluates to (folx/jvp.py:676-684 for the Jacobian, folx/hessian.py:115-175 for
    tr(J^T H J) on the pair of operands):
        J_y = fa J_a + fb J_b,   lap_y = fa lap_a + fb lap_b + faa |J_a|^2 + 2 fab J_a.J_b + fbb |J_b|^2."""
    Jy = fa[None] * Ja + fb[None] * Jb
    lap = fa * La + fb * Lb + faa * (Ja * Ja).sum(0) + 2 * fab * (Ja * Jb).sum(0) + fbb * (Jb * Jb).sum(0)
    return y, Jy, lap


def atan2_rule(a, Ja, La, b, Jb, Lb):
    """y = atan2(a, b) (``jax.lax.atan2``, folx/wrapped_functions.py:419): with r2 = a^2 + b^2,
    grad = (b, -a) / r2, Hessian = [[-2ab, a^2 - b^2], [a^2 - b^2, 2ab]] / r2^2."""
    a, b = np.broadcast_arrays(a, b)
    r2 = a * a + b * b
    return binary_hessian_rule(np.arctan2(a, b), b / r2, -a / r2, -2 * a * b / r2 ** 2, (a * a - b * b) / r2 ** 2,
                               2 * a * b / r2 ** 2, Ja, La, Jb, Lb)


def pow_rule(a, Ja, La, b, Jb, Lb):
    """y = a ** b for a > 0 with both operands variable (``jax.lax.pow``,
    folx/wrapped_functions.py:384)."""
    a, b = np.broadcast_arrays(a, b)
    y, la = a ** b, np.log(a)
    return binary_hessian_rule(y, b * y / a, y * la, b * (b - 1) * y / a ** 2, y / a * (1 + b * la), y * la * la,
                               Ja, La, Jb, Lb)


def rem_rule(a, Ja, La, b, Jb, Lb):
    """y = a - b trunc(a / b) (``jax.lax.rem``, folx/wrapped_functions.py:438): the quotient is
    piecewise constant, so the rule is linear."""
    a, b = np.broadcast_arrays(a, b)
    q = np.trunc(a / b)
    return a - b * q, Ja - q[None] * Jb, La - q * Lb


def add_rule(a, Ja, La, b, Jb, Lb, sign=1.0):
    """y = a +- b (LINEAR, folx/wrapped_functions.py:365-370)."""
    return a + sign * b, Ja + sign * Jb, La + sign * Lb


def minmax_rule(a, Ja, La, b, Jb, Lb, is_max=False):
    """``jax.lax.min`` / ``max`` of two triplets (LINEAR, folx/wrapped_functions.py:508-513):
    the selected operand's triplet passes through; at a tie each operand contributes half,
    which is how jax differentiates min / max."""
    a, b = np.broadcast_arrays(a, b)
    first = (a > b) if is_max else (a < b)
    w = np.where(first, 1.0, np.where(a == b, 0.5, 0.0)).astype(a.dtype)
    y = np.maximum(a, b) if is_max else np.minimum(a, b)
    return y, w * Ja + (1 - w) * Jb, w * La + (1 - w) * Lb


def scatter_rule(op, upd, tpos, mode):
    """Scatter of an updates triplet into an operand triplet at static positions
    (``sparse_scatter_jvp``'s arithmetic, folx/jvp.py:474-673, on dense Jacobians).

    op = (x (B, S_op), J (P, B, S_op), lap (B, S_op)), upd likewise with S_upd positions,
    ``tpos (S_upd,)`` the flat operand position each update element lands on (-1 = dropped).
    ``mode``: 'set' (a later element overwrites an earlier one), 'add', 'min', 'max'.
    Updates are applied one element at a time, in order."""
    x, J, L = (np.array(t, copy=True) for t in op)
    ux, uJ, uL = upd
    for e, p in enumerate(np.asarray(tpos).reshape(-1)):
        if p < 0:
            continue
        if mode == 'set':
            x[..., p], J[..., p], L[..., p] = ux[..., e], uJ[..., e], uL[..., e]
        elif mode == 'add':
            x[..., p] += ux[..., e]
            J[..., p] += uJ[..., e]
            L[..., p] += uL[..., e]
        else:
            x[..., p], J[..., p], L[..., p] = minmax_rule(
                x[..., p], J[..., p], L[..., p], ux[..., e], uJ[..., e], uL[..., e], is_max=(mode == 'max'))
    return x, J, L


def sum_rule(x, J, lap, axes, keepdims=False):
    """reduce_sum is linear (SUMMATION flag, folx/wrapped_functions.py:388-392): the same
    reduction is applied to x, J rows and lap (folx/jvp.py:104-106)."""
    ax = tuple(a % (x.ndim - 1) for a in np.atleast_1d(axes))
    xa = tuple(a + 1 for a in ax)
    ja = tuple(a + 2 for a in ax)
    return (
        x.sum(xa, keepdims=keepdims),
        J.sum(ja, keepdims=keepdims),
        lap.sum(xa, keepdims=keepdims),
    )


# --------------------------------------------------------------------------------------
# slogdet
# --------------------------------------------------------------------------------------


def slogdet_rule(A, J, lap):
    """Forward Laplacian of ``log|det A|`` from the dense Jacobian
    (folx/slogdet.py:296-317):

        M_c = A^-1 dA/dx_c,  d_c log|det A| = tr M_c,
        lap = tr(A^-1 lap_A) - sum_c tr(M_c M_c).

    A: (B, ..., n, n); J: (P, B, ..., n, n); lap: (B, ..., n, n).
    Returns sign (plain array), (logdet, J_logdet, lap_logdet).
    """
    sign, logdet = np.linalg.slogdet(A)
    Ainv = np.linalg.inv(A)
    M = np.einsum('...ij,p...jd->p...id', Ainv, J)
    jac = np.einsum('p...ii->p...', M)
    lap_out = np.einsum('...ji,...ij->...', Ainv, lap) - np.einsum(
        'p...id,p...di->...', M, M
    )
    return sign.astype(A.dtype), (logdet.astype(A.dtype), jac, lap_out)


def sparse_slogdet_rule(A, Jdata, lap, tables):
    """Forward Laplacian of ``log|det A|`` from rank-one factors of ``dA/dx_c``
    (folx/slogdet.py:182-246).  With ``dA/dx_c = sum_s e_{i_s} w_s^T`` (row factors
    restricted to the entries the coordinate touches) and
    ``W_c[s, t] = sum_l w_s[j_l] A^-1[j_l, i_t]``:

        d_c log|det A| = tr W_c,   lap = tr(A^-1 lap_A) - sum_c sum_st W_c[s,t] W_c[t,s].

    A, lap: (B, ..., n, n); Jdata: (k, B, ..., n, n) sparse rows; ``tables`` from
    ``oracle.index_algebra.slogdet_factor_tables``.  Returns sign and
    ``(logdet, jac (n_coords, B, ...), lap_out)``; the Jacobian rows belong to
    ``tables['coords']``.
    """
    take, cols, rows, per_entry = tables['take'], tables['cols'], tables['rows'], tables['per_entry']
    k = Jdata.shape[0]
    n, m = A.shape[-2:]
    batch = A.shape[:-2]
    sign, logdet = np.linalg.slogdet(A)
    Ainv = np.linalg.inv(A)
    C, R, Wd = take.shape
    Jb = np.broadcast_to(Jdata, (k, *A.shape))
    W = np.zeros((*batch, C, R, R), dtype=A.dtype)
    for c in range(C):
        for s in range(R):
            for t in range(R):
                acc = np.zeros(batch, dtype=A.dtype)
                if per_entry:
                    tot = np.zeros(batch, dtype=A.dtype)
                    for l in range(Wd):
                        pos = take[c, s, l]
                        if pos < k * n * m:
                            tt, rem = divmod(int(pos), n * m)
                            tot = tot + Jb[tt][..., rem // m, rem % m]
                    acc = tot * Ainv[..., cols[c, s, 0], rows[c, t]]
                else:
                    for l in range(Wd):
                        pos = take[c, s, l]
                        if pos < k * n * m:
                            tt, rem = divmod(int(pos), n * m)
                            acc = acc + Jb[tt][..., rem // m, rem % m] * Ainv[..., cols[c, s, l], rows[c, t]]
                W[..., c, s, t] = acc
    jac = np.moveaxis(np.einsum('...css->...c', W), -1, 0)
    lap_out = np.einsum('...ji,...ij->...', Ainv, lap) - np.einsum('...cst,...cts->...', W, W)
    return sign.astype(A.dtype), (logdet.astype(A.dtype), jac, lap_out)


def inv_rule(A, J, lap):
    """Forward Laplacian of ``C = A^-1`` (folx/linear_solve.py:114-145): with
    ``M_c = C dA/dx_c``,  ``d_c C = -M_c C``  and
    ``lap C = (2 sum_c M_c M_c - C lap_A) C``.
    A, lap: (B, ..., n, n); J: (P, B, ..., n, n)."""
    C = np.linalg.inv(A)
    M = np.einsum('...il,p...lj->p...ij', C, J)
    jac = -np.einsum('p...il,...lj->p...ij', M, C)
    inner = 2.0 * np.einsum('p...il,p...lj->...ij', M, M) - np.einsum('...il,...lj->...ij', C, lap)
    return C, jac, np.einsum('...il,...lj->...ij', inner, C)


def solve_rule(A, AJ, AL, b, bJ, bL):
    """Forward Laplacian of ``y = A^-1 b`` (folx/linear_solve.py:54-111):

        A d_c y = d_c b - d_c A y,     A lap_y = lap_b - lap_A y - 2 sum_c d_c A d_c y.

    A: (B, ..., n, n), b: (B, ..., n, m); either Jacobian/Laplacian pair may be None
    (constant operand) but not both.  Jacobians: (P, B, ..., n, *)."""
    assert AJ is not None or bJ is not None
    y = np.linalg.solve(A, b)
    P = (AJ if AJ is not None else bJ).shape[0]
    rhsJ = np.zeros((P, *y.shape), dtype=y.dtype)
    rhsL = np.zeros_like(y)
    if bJ is not None:
        rhsJ = rhsJ + bJ
        rhsL = rhsL + bL
    if AJ is not None:
        rhsJ = rhsJ - np.einsum('p...il,...lm->p...im', AJ, y)
        rhsL = rhsL - np.einsum('...il,...lm->...im', AL, y)
    yJ = np.linalg.solve(np.broadcast_to(A, (P, *A.shape)), rhsJ)
    if AJ is not None:
        rhsL = rhsL - 2.0 * np.einsum('p...il,p...lm->...im', AJ, yJ)
    return y, yJ, np.linalg.solve(A, rhsL)


# --------------------------------------------------------------------------------------
# Multi-head self attention
# --------------------------------------------------------------------------------------


def big_number(dtype) -> float:
    """Mask fill value (folx/experimental/pallas/attention/utils.py:210-220)."""
    return 1e40 if np.dtype(dtype) == np.float64 else 1e20


def mhsa_forward(q, k, v, mask=None, e=None):
    """softmax(q k^T (+ e)) v with padded-sequence masking and no 1/sqrt(d) inside
    (folx/experimental/pallas/attention/mhsa.py:79-94, mhsea.py:80-97).
    q, k, v: (B, n, H, d); e: (B, n, H, n)."""
    B, n, H, d = q.shape
    if mask is None:
        mask = np.ones((B, n), dtype=bool)
    sq = mask[:, :, None, None] & mask[:, None, None, :]
    s = np.einsum('bihd,bjhd->bihj', q, k)
    if e is not None:
        s = s + e
    s = np.where(sq, s, -big_number(s.dtype))
    s = s - s.max(-1, keepdims=True)
    e = np.exp(s)
    p = e / e.sum(-1, keepdims=True)
    return np.einsum('bihj,bjhd->bihd', p, v), p


def mhsa_rule(q, qJ, qL, k, kJ, kL, v, vJ, vL, mask=None, input_mask=None, e=None, eJ=None, eL=None):
    """Forward Laplacian of masked multi-head self attention, optionally with an additive
    edge bias ``e (B, n, H, n)`` on the scores (``s = q k^T + e``): the edge term enters
    ``s'_c`` and the direct Laplacian part linearly and has no second-order contribution
    (folx/experimental/pallas/attention/forward_laplacian.py:663-704).  Its Jacobian rows
    are zeroed for inactive coordinates only (:649).


    Specification: folx/experimental/pallas/attention/forward_laplacian.py:212-346 (einsum
    form) and :349-487 (kernel form); the algebra below is the factored form the same
    file uses for the edge-bias variant (:663-704) with the edge term removed:

        s'_c = q'_c k^T + q k'_c^T          p'_c = p * (s'_c - rowsum(p * s'_c))
        o'_c = p v'_c + p'_c v
        lap_o = [same with the Laplacians in place of the c-derivatives]
              + ( sum_c p'_c * (s'_c - rowsum(p s'_c))
                  + p * (S - sum_c rowsum(p'_c s'_c) - rowsum(p S)) ) v
              + 2 sum_c p'_c v'_c,           S = 2 sum_c q'_c k'_c^T

    Masking (:231-241): Jacobian rows are zeroed where the coordinate is inactive
    (``input_mask[p, b]`` False) or the electron is padding (``mask[b, i]`` False);
    Laplacians are zeroed for padding electrons; scores of padded pairs are set to
    ``-big_number`` before the softmax.  Rows of padding queries carry no meaning (the
    reference's tests mask them out before comparing, test_attention.py:80-100).

    Shapes: q/k/v (B, n, H, d); *J (P, B, n, H, d); *L (B, n, H, d);
    mask (B, n) bool; input_mask (P, B) bool.
    """
    B, n, H, d = q.shape
    P = qJ.shape[0]
    if mask is None:
        mask = np.ones((B, n), dtype=bool)
    if input_mask is None:
        input_mask = np.ones((P, B), dtype=bool)
    mask = mask.astype(bool)
    input_mask = input_mask.astype(bool)
    cm = input_mask[:, :, None, None, None] & mask[None, :, :, None, None]
    em = mask[:, :, None, None]
    qJ, kJ, vJ = (np.where(cm, a, 0.0) for a in (qJ, kJ, vJ))
    qL, kL, vL = (np.where(em, a, 0.0) for a in (qL, kL, vL))

    o, p = mhsa_forward(q, k, v, mask, e)

    sJ = np.einsum('pbihd,bjhd->pbihj', qJ, k) + np.einsum('bihd,pbjhd->pbihj', q, kJ)
    if e is not None:
        sJ = sJ + np.where(input_mask[:, :, None, None, None], eJ, 0.0)
    rJ = (p[None] * sJ).sum(-1, keepdims=True)
    pJ = p[None] * (sJ - rJ)
    oJ = np.einsum('bihj,pbjhd->pbihd', p, vJ) + np.einsum('pbihj,bjhd->pbihd', pJ, v)

    sL = np.einsum('bihd,bjhd->bihj', qL, k) + np.einsum('bihd,bjhd->bihj', q, kL)
    if e is not None:
        sL = sL + eL
    pL = p * (sL - (p * sL).sum(-1, keepdims=True))
    oL = np.einsum('bihj,bjhd->bihd', p, vL) + np.einsum('bihj,bjhd->bihd', pL, v)

    S = 2 * np.einsum('pbihd,pbjhd->bihj', qJ, kJ)
    pI = (pJ * (sJ - rJ)).sum(0) + p * (
        S - (pJ * sJ).sum((0, -1))[..., None] - (p * S).sum(-1, keepdims=True)
    )
    oL = oL + np.einsum('bihj,bjhd->bihd', pI, v)
    oL = oL + 2 * np.einsum('pbihj,pbjhd->bihd', pJ, vJ)
    return o, oJ, oL

"""Pins oracle.rules against checks that do not retype its formulas: torch fp64 autograd
(jvp-of-jvp for activations, full Hessian traces for the composite rules), numpy.linalg
closed forms for slogdet, and the masked-attention cases of the reference's own test
(test/experimental/pallas/test_attention.py:320-326)."""

import numpy as np
import pytest
import torch

from bruteforce import brute_force, plain
from oracle import backend as ob
from oracle import rules

RTOL, ATOL = 2e-5, 1e-10  # the reference's own bar (test/laplacian_testcase.py:16-20)


def _close(a, b, rtol=RTOL, atol=ATOL):
    np.testing.assert_allclose(a, b, rtol=rtol, atol=atol)


POSITIVE = {'log', 'sqrt', 'rsqrt', 'log1p', 'reciprocal', 'cbrt'}
UNIT = {'asin', 'acos', 'atanh', 'erf_inv'}      # domain (-1, 1)
PLAIN_NAME = {'neg': 'negative', 'identity': None, 'asin': 'arcsin', 'acos': 'arccos', 'atan': 'arctan',
              'asinh': 'arcsinh', 'acosh': 'arccosh', 'atanh': 'arctanh'}


@pytest.mark.parametrize('name', sorted(rules.ACTIVATIONS))
def test_activation_closed_forms_vs_autograd(name):
    rng = np.random.default_rng(0)
    x = rng.normal(size=64) * 2
    if name in POSITIVE:
        x = np.abs(x) + 0.1
    if name in UNIT:
        x = rng.uniform(-0.9, 0.9, size=64)
    if name == 'acosh':
        x = np.abs(x) + 1.1
    if name in ('lgamma', 'digamma'):   # positive arguments and negative ones away from the poles
        x = np.concatenate([rng.uniform(0.3, 7.0, size=40), rng.integers(-3, 0, size=24) + rng.uniform(0.25, 0.75, size=24)])
    tname = PLAIN_NAME.get(name, name)
    f = (lambda t: t) if tname is None else getattr(plain, tname)
    xt = torch.tensor(x, dtype=torch.float64)
    ones = torch.ones_like(xt)
    df = lambda t: torch.func.jvp(f, (t,), (ones,))[1]
    d1 = df(xt)
    d2 = torch.func.jvp(df, (xt,), (ones,))[1]
    y, g1, g2 = rules.ACTIVATIONS[name](x)
    _close(y, f(xt).numpy())
    _close(g1, d1.numpy())
    _close(g2, d2.numpy(), atol=1e-9)


@pytest.mark.parametrize('c', [2.5, -0.5, 1.0 / 3.0])
def test_pow_constant_exponent(c):
    x = np.random.default_rng(1).uniform(0.2, 3.0, size=32)
    xt = torch.tensor(x, dtype=torch.float64)
    ones = torch.ones_like(xt)
    f = lambda t: t**c
    df = lambda t: torch.func.jvp(f, (t,), (ones,))[1]
    y, J, L = rules.elementwise_rule('pow', x, np.ones((1, 32)), np.zeros(32), c)
    _close(y, f(xt).numpy()), _close(J[0], df(xt).numpy())
    _close(L, torch.func.jvp(df, (xt,), (ones,))[1].numpy(), atol=1e-9)


def test_integer_pow():
    x = np.linspace(0.5, 2, 7)
    for n in (2, 3, -1, -2):
        y, d1, d2 = rules.integer_pow(x, n)
        _close(y, x**n)
        _close(d1, n * x ** (n - 1))
        _close(d2, n * (n - 1) * x ** (n - 2))


def _run_oracle(fn, x):
    out = fn(ob, ob.init_state(x, dtype=np.float64))
    return out.x, out.J, out.lap


def _check(fn, x, rtol=RTOL, atol=1e-9):
    y, J, L = _run_oracle(fn, x)
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x)
    _close(y, by, rtol, atol)
    _close(J, bJ, rtol, atol)
    _close(L, bL, rtol, atol)


def test_mlp_vs_bruteforce():
    # same structure as test/test_composite.py:13-43 (tanh MLP, summed)
    rng = np.random.default_rng(1)
    Ws = [(rng.normal(size=(12, 12)) / 3, rng.normal(size=12)) for _ in range(3)]

    def mlp(xp, x):
        for W, b in Ws:
            x = xp.tanh(xp.dot(x, W, b))
        return xp.sum(x)

    _check(mlp, rng.normal(size=(3, 12)))


def test_silu_mlp_nodewise_vs_bruteforce():
    # README example shape in miniature: nodes pass through the MLP independently
    rng = np.random.default_rng(2)
    Ws = [rng.normal(size=(4, 6)) / 2, rng.normal(size=(6, 6)) / 2, rng.normal(size=(6, 1))]

    def f(xp, x):
        for W in Ws[:-1]:
            x = xp.silu(xp.dot(x, W))
        return xp.sum(xp.dot(x, Ws[-1]))

    _check(f, rng.normal(size=(2, 5, 4)))


@pytest.mark.parametrize('op', ['multiply', 'divide', 'add', 'subtract'])
def test_binary_rules_vs_bruteforce(op):
    rng = np.random.default_rng(3)
    W1, W2 = rng.normal(size=(6, 5)), rng.normal(size=(6, 5))

    def f(xp, x):
        a = xp.tanh(xp.dot(x, W1))
        b = xp.add(xp.exp(xp.dot(x, W2) * 0.3 if xp is plain else xp.multiply(xp.dot(x, W2), 0.3)), 0.5)
        return getattr(xp, op)(a, b)

    _check(f, rng.normal(size=(2, 6)))


def test_binary_broadcast_and_reductions_vs_bruteforce():
    # layer-norm built from primitives: mean / sub / square / rsqrt / mul with broadcasting
    rng = np.random.default_rng(4)
    g = rng.normal(size=8)

    def ln(xp, x):
        mu = xp.mean(x, axis=-1, keepdims=True)
        c = xp.subtract(x, mu)
        var = xp.mean(xp.square(c), axis=-1, keepdims=True)
        y = xp.multiply(c, xp.rsqrt(xp.add(var, 1e-5)))
        return xp.multiply(y, g)

    _check(ln, rng.normal(size=(2, 3, 8)))


def test_indexing_ops_vs_bruteforce():
    rng = np.random.default_rng(5)
    R = rng.normal(size=(2, 3))

    def feats(xp, r):  # r (4, 3): electron-nucleus vectors and distances
        d = xp.subtract(xp.expand_dims(r, 1), R)  # (4, 2, 3)
        dist = xp.sqrt(xp.sum(xp.square(d), axis=-1))  # (4, 2)
        f = xp.concatenate([xp.reshape(d, (4, 6)), dist], axis=-1)  # (4, 8)
        f = xp.transpose(f, (1, 0))
        return xp.getitem(f, (slice(1, 7),))

    _check(feats, rng.normal(size=(2, 4, 3)))


@pytest.mark.parametrize('n', [1, 2, 4, 6])
def test_slogdet_vs_bruteforce(n):
    # shapes of test/test_layers.py:341-396 (small matrices through a tanh layer)
    rng = np.random.default_rng(6)
    W = rng.normal(size=(5, n * n))

    def f(xp, x):
        A = xp.reshape(xp.tanh(xp.dot(x, W)), (n, n))
        return xp.slogdet(A)[1]

    _check(f, rng.normal(size=(3, 5)), rtol=1e-4 if n == 6 else RTOL, atol=1e-8)


@pytest.mark.parametrize('n', [2, 3])
def test_slogdet_vs_cofactor_expansion(n):
    """log|det| written as an explicit polynomial (no linalg call in the brute force), so
    the check does not lean on torch's derivative formulas for det / slogdet."""
    rng = np.random.default_rng(16)
    W = rng.normal(size=(4, n * n))

    def det_poly(A):
        if n == 2:
            return A[0, 0] * A[1, 1] - A[0, 1] * A[1, 0]
        return (
            A[0, 0] * (A[1, 1] * A[2, 2] - A[1, 2] * A[2, 1])
            - A[0, 1] * (A[1, 0] * A[2, 2] - A[1, 2] * A[2, 0])
            + A[0, 2] * (A[1, 0] * A[2, 1] - A[1, 1] * A[2, 0])
        )

    def f(xp, x):
        A = xp.reshape(xp.tanh(xp.dot(x, W)), (n, n))
        if xp is plain:
            return torch.log(torch.abs(det_poly(A)))
        return xp.slogdet(A)[1]

    _check(f, rng.normal(size=(3, 4)), atol=1e-8)


def test_slogdet_closed_forms():
    rng = np.random.default_rng(7)
    B, n, P = 4, 5, 3
    # diagonal A(x): log|det| = sum log|a_ii|, derivative rows only on the diagonal
    a = rng.uniform(0.5, 2.0, size=(B, n)) * rng.choice([-1, 1], size=(B, n))
    A = np.zeros((B, n, n))
    A[:, range(n), range(n)] = a
    Jd = rng.normal(size=(P, B, n))
    J = np.zeros((P, B, n, n))
    J[:, :, range(n), range(n)] = Jd
    Ld = rng.normal(size=(B, n))
    L = np.zeros((B, n, n))
    L[:, range(n), range(n)] = Ld
    sign, (ld, Jo, Lo) = rules.slogdet_rule(A, J, L)
    _close(sign, np.prod(np.sign(a), -1))
    _close(ld, np.log(np.abs(a)).sum(-1))
    _close(Jo, (Jd / a[None]).sum(-1))
    _close(Lo, (Ld / a).sum(-1) - ((Jd / a[None]) ** 2).sum((0, -1)))
    # swapping two rows flips the sign and nothing else
    A2 = rng.normal(size=(B, n, n))
    J2, L2 = rng.normal(size=(P, B, n, n)), rng.normal(size=(B, n, n))
    perm = [1, 0, 2, 3, 4]
    s1, (l1, j1, p1) = rules.slogdet_rule(A2, J2, L2)
    s2, (l2, j2, p2) = rules.slogdet_rule(A2[:, perm], J2[:, :, perm], L2[:, perm])
    _close(s2, -s1), _close(l2, l1), _close(j2, j1), _close(p2, p1, atol=1e-9)


@pytest.mark.parametrize('n,H,d,valid', [(1, 1, 1, 1), (4, 2, 3, 4), (5, 2, 3, 2)])
def test_mhsa_vs_bruteforce(n, H, d, valid):
    """softmax(q k^T) v where q, k, v are random linear maps of the 3n inputs; the last
    case pads the sequence as test_attention.py:323-326 does (max_sequence < n)."""
    rng = np.random.default_rng(8)
    n_in = 3 * n
    Wq, Wk, Wv = (rng.normal(size=(n_in, n * H * d)) / np.sqrt(n_in) for _ in range(3))
    mask = np.zeros(n, dtype=bool)
    mask[:valid] = True
    in_mask = np.zeros(n_in, dtype=bool)
    in_mask[: 3 * valid] = True

    def f(xp, x):
        x = xp.reshape(x, (n_in,))
        q, k, v = (xp.reshape(xp.tanh(xp.dot(x, W)), (n, H, d)) for W in (Wq, Wk, Wv))
        if xp is plain:
            return xp.multi_head_self_attention(q, k, v, mask)
        B = q.B
        return xp.multi_head_self_attention(
            q, k, v, np.broadcast_to(mask, (B, n)), np.broadcast_to(in_mask[:, None], (n_in, B))
        )

    x = rng.normal(size=(2, n_in))
    # padded electrons' coordinates are inactive inputs: zero weights in the forward
    # Laplacian (folx/interpreter.py:319 ``weights=``), frozen in the brute force
    w = np.broadcast_to(in_mask.astype(np.float64), (n_in,))
    out = f(ob, ob.init_state(x, weights=w, dtype=np.float64))
    y, J, L = out.x, out.J, out.lap

    def f_plain(t):
        t = torch.where(torch.as_tensor(in_mask), t, t.detach())
        return f(plain, t)

    by, bJ, bL = brute_force(f_plain, x)
    m = mask
    _close(y[:, m], by[:, m], atol=1e-9)
    _close(J[:, :, m], bJ[:, :, m], atol=1e-9)
    _close(L[:, m], bL[:, m], rtol=1e-5, atol=1e-8)


def test_mhsa_masking_zeroes_inactive_rows():
    rng = np.random.default_rng(9)
    P, B, n, H, d = 6, 2, 4, 1, 2
    t = lambda *s: rng.normal(size=s)
    args = [t(B, n, H, d), t(P, B, n, H, d), t(B, n, H, d)] * 3
    in_mask = np.ones((P, B), dtype=bool)
    in_mask[3:] = False
    o, oJ, oL = rules.mhsa_rule(*args, None, in_mask)
    assert np.all(oJ[3:] == 0)
    # inactive coordinates do not contribute to the Laplacian either
    args2 = [a.copy() for a in args]
    for i in (1, 4, 7):
        args2[i][3:] = 123.0
    o2, oJ2, oL2 = rules.mhsa_rule(*args2, None, in_mask)
    _close(oL, oL2)
    _close(oJ, oJ2)


@pytest.mark.parametrize('n,H,d,valid', [(1, 1, 1, 1), (4, 2, 3, 4), (5, 2, 3, 3)])
def test_mhsea_vs_bruteforce(n, H, d, valid):
    """softmax(q k^T + e) v with an input-dependent edge bias, incl. a padded sequence
    (test/experimental/pallas/test_attention.py:389-459)."""
    rng = np.random.default_rng(18)
    n_in = 3 * n
    Wq, Wk, Wv = (rng.normal(size=(n_in, n * H * d)) / np.sqrt(n_in) for _ in range(3))
    We = rng.normal(size=(n_in, n * H * n)) / np.sqrt(n_in)
    mask = np.zeros(n, dtype=bool)
    mask[:valid] = True
    in_mask = np.zeros(n_in, dtype=bool)
    in_mask[: 3 * valid] = True

    def f(xp, x):
        x = xp.reshape(x, (n_in,))
        q, k, v = (xp.reshape(xp.tanh(xp.dot(x, W)), (n, H, d)) for W in (Wq, Wk, Wv))
        e = xp.reshape(xp.sin(xp.dot(x, We)), (n, H, n))
        if xp is plain:
            return xp.multi_head_self_attention(q, k, v, mask, None, e)
        B = q.B
        return xp.multi_head_self_attention(
            q, k, v, np.broadcast_to(mask, (B, n)), np.broadcast_to(in_mask[:, None], (n_in, B)), e)

    x = rng.normal(size=(2, n_in))
    out = f(ob, ob.init_state(x, weights=in_mask.astype(np.float64), dtype=np.float64))

    def f_plain(t):
        return f(plain, torch.where(torch.as_tensor(in_mask), t, t.detach()))

    by, bJ, bL = brute_force(f_plain, x)
    m = mask
    _close(out.x[:, m], by[:, m], atol=1e-9)
    _close(out.J[:, :, m], bJ[:, :, m], atol=1e-9)
    _close(out.lap[:, m], bL[:, m], rtol=1e-5, atol=1e-8)


def test_dot_two_rule_vs_autograd_and_mul_sum():
    """rules.dot_two_rule: (i) equals the multiply-and-sum decomposition built from mul_rule and
    sum_rule (both pinned by AD above), (ii) the Hessian trace of u(x) @ v(x) by torch AD."""
    import torch

    rng = np.random.default_rng(3)
    P, B, I, Kc, J = 5, 2, 3, 4, 6
    a, La, b, Lb = (rng.normal(size=s) for s in ((B, I, Kc), (B, I, Kc), (B, Kc, J), (B, Kc, J)))
    Ja, Jb = rng.normal(size=(P, B, I, Kc)), rng.normal(size=(P, B, Kc, J))
    y, Jy, ly = rules.dot_two_rule(a, Ja, La, b, Jb, Lb)
    bt = np.swapaxes
    m = rules.mul_rule(a[:, :, None, :], Ja[:, :, :, None, :], La[:, :, None, :],
                       bt(b, -1, -2)[:, None], bt(Jb, -1, -2)[:, :, None], bt(Lb, -1, -2)[:, None])
    sy, sJ, sl = rules.sum_rule(*m, axes=(2,))
    np.testing.assert_allclose(y, sy, rtol=1e-12)
    np.testing.assert_allclose(Jy, sJ, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(ly, sl, rtol=1e-12, atol=1e-12)
    # AD: f(x) = tanh(x A) @ sin(x C) for x in R^5, with the operands' triplets from the chain rule
    n = 5
    A, C = rng.normal(size=(n, I * Kc)), rng.normal(size=(n, Kc * J))
    x = torch.tensor(rng.normal(size=n), dtype=torch.float64)
    At, Ct = torch.tensor(A), torch.tensor(C)
    u = lambda t: torch.tanh(t @ At).reshape(I, Kc)
    v = lambda t: torch.sin(t @ Ct).reshape(Kc, J)
    f = lambda t: (u(t) @ v(t)).reshape(-1)
    jac = lambda g: torch.autograd.functional.jacobian(g, x)
    hess_tr = lambda g, m_: torch.stack([torch.autograd.functional.hessian(lambda t: g(t).reshape(-1)[i], x).trace()
                                         for i in range(m_)])
    tri = lambda g, shp: (g(x).numpy()[None], np.moveaxis(jac(lambda t: g(t).reshape(-1)).numpy(), -1, 0).reshape(n, 1, *shp),
                          hess_tr(g, int(np.prod(shp))).numpy().reshape(1, *shp))
    ua, vb = tri(u, (I, Kc)), tri(v, (Kc, J))
    got = rules.dot_two_rule(*ua, *vb)
    want = tri(lambda t: u(t) @ v(t), (I, J))
    for g_, w_ in zip(got, want):
        np.testing.assert_allclose(g_, w_, rtol=1e-9, atol=1e-10)


def test_where_broadcasts_operands_of_different_rank_like_numpy():
    """The oracle backend's ``where`` with a condition of rank 5, one operand of rank 5 and one of rank 1 (aligned on the
    right, behind the walker axis) against AD through ``torch.where``."""
    from bruteforce import brute_force, plain
    from oracle import backend as ob

    cond = np.array([True, False]).reshape(2, 1, 1, 1, 1)

    def f(xp, x):
        a = xp.add(xp.tanh(xp.reshape(xp.getitem(x, slice(0, 2)), (2, 1, 1, 1, 1))), 2.0)
        r = xp.add(xp.reshape(xp.cos(xp.getitem(x, slice(2, 5))), (3,)), 2.0)
        return xp.where(cond, a, r), xp.where(cond, 0.5, r), xp.where(cond[:, 0], a, np.float64(1.5))

    x = np.random.default_rng(0).normal(size=(2, 5))
    got = f(ob, ob.init_state(x, dtype=np.float64))
    for i, g in enumerate(got):
        y, J, L = brute_force(lambda t, i=i: f(plain, t)[i], x)
        assert g.x.shape == y.shape
        np.testing.assert_allclose(g.x, y, rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(g.J, J.reshape(g.J.shape), rtol=1e-12, atol=1e-13)
        np.testing.assert_allclose(g.lap, L, rtol=1e-12, atol=1e-13)

"""Pins the oracle's inverse, linear-solve and sparse-slogdet rules.

* inverse / solve: fp64 Hessian traces by AD of an adjugate-over-determinant inverse
  (pure arithmetic, no linalg derivative formula involved), on the cases of the
  reference's test/test_layers.py:443-499, plus 1x1 / diagonal closed forms.
* sparse slogdet: the path choices the reference's tests expect
  (test/test_layers.py:341-421: which Jacobian structures take the rank-one shortcut, and
  the table shape of the element-sparse case), and equality with the dense slogdet rule,
  which is itself pinned by brute force.
"""

import numpy as np
import pytest

from bruteforce import brute_force, plain
from oracle import backend as ob
from oracle import index_algebra as ia
from oracle import rules

RTOL = 2e-5


def _close(a, b, rtol=RTOL, atol=1e-9):
    np.testing.assert_allclose(a, b, rtol=rtol, atol=atol)


def _check(fn, x, rtol=RTOL, atol=1e-8):
    out = fn(ob, ob.init_state(x, dtype=np.float64))
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x)
    _close(out.x, by, rtol, atol)
    _close(out.J, bJ, rtol, atol)
    _close(out.lap, bL, rtol, atol)


def _matrix(xp, x, W, n, lead=()):
    """n I + tanh(x W) reshaped to (*lead, n, n): well conditioned, depends on every input."""
    A = xp.reshape(xp.tanh(xp.dot(xp.reshape(x, (-1,)), W)), (*lead, n, n))
    return xp.add(A, n * np.eye(n))


@pytest.mark.parametrize('n', [1, 2, 4])
def test_inv_vs_bruteforce(n):
    rng = np.random.default_rng(21)
    W = rng.normal(size=(3 * n, n * n))
    _check(lambda xp, x: xp.inv(_matrix(xp, x, W, n)), rng.normal(size=(2, n, 3)))


def test_inv_closed_form_1x1():
    # C = 1/a: d C = -J / a^2, lap C = 2 sum J^2 / a^3 - L / a^2
    rng = np.random.default_rng(22)
    a = rng.uniform(0.5, 2.0, size=(3, 1, 1))
    J, L = rng.normal(size=(4, 3, 1, 1)), rng.normal(size=(3, 1, 1))
    C, Cj, Cl = rules.inv_rule(a, J, L)
    _close(C, 1 / a)
    _close(Cj, -J / a**2)
    _close(Cl, 2 * (J**2).sum(0) / a**3 - L / a**2)


SOLVE_CASES = ['matrix varies, vector rhs', 'matrix varies, matrix rhs', 'both vary', 'rhs varies',
               'batched matrix']


@pytest.mark.parametrize('case', SOLVE_CASES)
def test_solve_vs_bruteforce(case):
    # the five cases of test/test_layers.py:443-480 at n = 3
    n = 3
    rng = np.random.default_rng(23)
    W = rng.normal(size=(3 * n, n * n))
    Wb = rng.normal(size=(3 * n, 2 * n * n))
    A_const = n * np.eye(n) + np.tril(rng.normal(size=(n, n)), -1)
    b_vec, b_mat = rng.normal(size=(n,)), rng.normal(size=(n, 2))

    def f(xp, x):
        rhs = xp.sum(xp.tanh(x), axis=-1)
        if case == 'matrix varies, vector rhs':
            return xp.solve(_matrix(xp, x, W, n), b_vec)
        if case == 'matrix varies, matrix rhs':
            return xp.solve(_matrix(xp, x, W, n), b_mat)
        if case == 'both vary':
            return xp.solve(_matrix(xp, x, W, n), rhs)
        if case == 'rhs varies':
            return xp.solve(A_const, rhs)
        return xp.solve(_matrix(xp, x, Wb, n, lead=(2,)), rhs)

    _check(f, rng.normal(size=(2, n, 3)))


def test_solve_diagonal_closed_form():
    # diagonal constant A: y_i = b_i / a_i, and the rule is linear in b
    rng = np.random.default_rng(24)
    B, n, m, P = 3, 4, 2, 5
    a = rng.uniform(0.5, 2.0, size=(B, n))
    A = np.zeros((B, n, n))
    A[:, range(n), range(n)] = a
    b, bJ, bL = rng.normal(size=(B, n, m)), rng.normal(size=(P, B, n, m)), rng.normal(size=(B, n, m))
    y, yJ, yL = rules.solve_rule(A, None, None, b, bJ, bL)
    _close(y, b / a[..., None]), _close(yJ, bJ / a[None, ..., None]), _close(yL, bL / a[..., None])


# ---------------------------------------------------------------------------------------
# sparse slogdet
# ---------------------------------------------------------------------------------------


def _slater_mask(mode, n=6, d=3):
    """Jacobian masks (k, n, n) of the matrices built in test/test_layers.py:341-384: a
    row (or column) of A depends on the d coordinates of one particle."""
    if mode in ('row_sparse', 'columns'):
        m = np.empty((d, n, n), dtype=np.int64)
        for t in range(d):
            for i in range(n):
                m[t, i, :] = d * i + t
        return m if mode == 'row_sparse' else np.swapaxes(m, -1, -2).copy()
    if mode in ('two_rows', 'two_columns'):
        # A + roll(A, 1): row i depends on particles i and i - 1
        m = np.empty((2 * d, n, n), dtype=np.int64)
        for i in range(n):
            deps = sorted([d * i + t for t in range(d)] + [d * ((i - 1) % n) + t for t in range(d)])
            for r, v in enumerate(deps):
                m[r, i, :] = v
        return m if mode == 'two_rows' else np.swapaxes(m, -1, -2).copy()
    if mode == 'shared_rows':
        # A + x.sum(): every entry depends on every coordinate
        return np.broadcast_to(np.arange(n * d).reshape(n * d, 1, 1), (n * d, n, n)).copy()
    raise ValueError(mode)


@pytest.mark.parametrize('mode,expect_fast', [('row_sparse', True), ('two_rows', True), ('columns', True),
                                              ('two_columns', True), ('shared_rows', False)])
def test_sparse_slogdet_path_choice(mode, expect_fast):
    """Which structures take the shortcut (test/test_layers.py:341-398)."""
    mask = _slater_mask(mode)
    plan = ia.slogdet_plan(mask, mask.shape[0], (6, 6), int(mask.max()))
    assert (plan is not None) is expect_fast
    if mode == 'row_sparse':
        tables, transposed = plan
        assert not transposed and not tables['per_entry']
        assert tables['take'].shape == (18, 1, 6)
    if mode == 'columns':
        tables, transposed = plan
        # rows of A^T; the untransposed entry factors would cost 18 * 6 * 6
        assert transposed and tables['take'].shape == (18, 1, 6)


def test_sparse_slogdet_batched_mask_shared():
    # (mol, det, elec, orb) stack as in the 'batched' case: same mask at every batch position
    mask = _slater_mask('row_sparse')
    stacked = np.broadcast_to(mask[:, None, None], (3, 1, 2, 6, 6))
    got = ia.slogdet_entry_mask(stacked, 3, (1, 2, 6, 6), False)
    np.testing.assert_array_equal(got, mask)
    other = stacked.copy()
    other[0, 0, 1, 0, 0] = 17
    assert ia.slogdet_entry_mask(other, 3, (1, 2, 6, 6), False) is None
    # a mask that does not spell out every axis cannot be transposed
    assert ia.slogdet_entry_mask(mask[0, :1], 1, (6, 6), True) is None
    assert ia.slogdet_entry_mask(mask[0, :1], 1, (6, 6), False).shape == (1, 6, 6)
    assert ia.slogdet_entry_mask(None, 3, (6, 6), False) is None


def test_sparse_slogdet_element_sparse_tables():
    """test/test_layers.py:400-421: A = 2 I + tanh(x)[perm], every coordinate touches one
    entry per row -> n factors of one entry each per coordinate, tables of shape (n, n, 1)."""
    n = 6
    perm = np.stack([np.roll(np.arange(n), s) for s in range(n)])
    plan = ia.slogdet_plan(perm[None], 1, (n, n), n - 1)
    assert plan is not None
    tables, transposed = plan
    assert tables['take'].shape == (n, n, 1)
    assert not transposed


@pytest.mark.parametrize('mode', ['row_sparse', 'two_rows', 'columns', 'two_columns', 'element', 'ragged'])
@pytest.mark.parametrize('per_entry', [False, True])
def test_sparse_slogdet_rule_equals_dense_rule(mode, per_entry):
    rng = np.random.default_rng(25)
    n, B = 6, 3
    if mode == 'element':
        mask = np.stack([np.roll(np.arange(n), s) for s in range(n)])[None]
    elif mode == 'ragged':
        # random support with holes and a coordinate repeated across tangent rows
        mask = rng.integers(-1, 5, size=(2, n, n))
        mask[1][mask[1] == mask[0]] = -1
    else:
        mask = _slater_mask(mode)
    k = mask.shape[0]
    A = rng.normal(size=(B, 2, n, n)) + 2 * np.eye(n)
    Jd = rng.normal(size=(k, B, 2, n, n)) * (mask >= 0)[:, None, None]
    L = rng.normal(size=(B, 2, n, n))
    cost, tables = ia.slogdet_factor_tables(mask, per_entry)
    sign, (ld, jac, lap) = rules.sparse_slogdet_rule(A, Jd, L, tables)
    dense = ia.dense_array(Jd, np.broadcast_to(mask[:, None], (k, 2, n, n)))
    sign0, (ld0, jac0, lap0) = rules.slogdet_rule(A, dense, L)
    _close(sign, sign0), _close(ld, ld0), _close(lap, lap0)
    full = np.zeros_like(jac0)
    full[tables['coords']] = jac
    _close(full, jac0)
    C, R, Wd = tables['take'].shape
    assert cost == C * R * R * (1 if per_entry else Wd)

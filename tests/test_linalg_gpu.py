"""GPU parity of the inverse, linear-solve and sparse-slogdet entry points against the fp64
oracle on the same seeded fp32 inputs (kernel level, through libfolx_hip.so), and of the
rules built on them against the dense oracle (model level; the cases of the reference's
test/test_layers.py:341-499)."""

import numpy as np
import pytest
import torch

from oracle import backend as ob
from oracle import index_algebra as oia
from oracle import rules

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype).cuda()


def f64(*arrs):
    return [None if a is None else np.asarray(a, dtype=np.float64) for a in arrs]


def rand(rng, *shape):
    return rng.normal(size=shape).astype(np.float32)


def well_conditioned(rng, *lead, n):
    """Random matrices with a dominant diagonal: condition numbers of a few units, so the
    strict parity bars apply without an amplification factor."""
    return (rand(rng, *lead, n, n) / np.sqrt(n) + 2.0 * np.eye(n, dtype=np.float32)).astype(np.float32)


def close(got, ref, what, lap=False, amp=1.0):
    got = got.detach().cpu().numpy().astype(np.float64)
    scale = float(np.abs(ref).max())
    if lap:
        np.testing.assert_allclose(got, ref, rtol=1e-4 * amp, atol=(1e-5 + 1e-5 * scale) * amp, err_msg=what)
    else:
        np.testing.assert_allclose(got, ref, rtol=1e-5 * amp, atol=2e-6 * scale * amp, err_msg=what)


@pytest.mark.parametrize('n,P,lead', [(1, 3, (4,)), (2, 5, (3, 2)), (5, 7, (6,)), (8, 24, (4, 3)),
                                      (16, 96, (5, 4)), (32, 20, (3, 2)), (11, 4, (7,)), (4, 0, (3,))])
def test_inv(n, P, lead):
    from folx_amd import kernels as K

    print(f'case inv n={n} P={P} lead={lead}', flush=True)
    rng = np.random.default_rng(40)
    A = well_conditioned(rng, *lead, n=n)
    J, L = rand(rng, P, *lead, n, n), rand(rng, *lead, n, n)
    C, CJ, CL = rules.inv_rule(*f64(A, J, L))
    gC, gJ, gL = K.inv(dev(A), dev(J), dev(L))
    close(gC, C, 'inverse')
    if P:
        close(gJ, CJ, 'jacobian')
    # the Laplacian sums P products of three matrices: a few more roundings than a value
    close(gL, CL, 'laplacian', lap=True)


def test_inv_pivoting():
    """A permuted diagonal needs a row exchange at every step; the result is exact."""
    from folx_amd import kernels as K

    rng = np.random.default_rng(41)
    n, B = 8, 5
    perm = rng.permutation(n)
    d = rng.uniform(0.5, 2.0, size=(B, n)).astype(np.float32)
    A = np.zeros((B, n, n), np.float32)
    A[:, np.arange(n), perm] = d
    J, L = rand(rng, 3, B, n, n), rand(rng, B, n, n)
    C, CJ, CL = rules.inv_rule(*f64(A, J, L))
    gC, gJ, gL = K.inv(dev(A), dev(J), dev(L))
    close(gC, C, 'inverse'), close(gJ, CJ, 'jacobian'), close(gL, CL, 'laplacian', lap=True)


SOLVE_CASES = [
    # n, m, P, lead, A varies, b varies
    (1, 1, 3, (4,), True, True),
    (5, 1, 7, (6,), True, False),
    (5, 2, 7, (6,), True, True),
    (5, 1, 7, (3, 2), False, True),
    (8, 8, 12, (4,), True, True),
    (16, 1, 48, (5, 2), True, True),
    (16, 3, 9, (5,), False, True),
    (7, 20, 4, (3,), True, True),     # more right-hand sides than unknowns
    (32, 1, 10, (4,), True, True),
    (32, 32, 5, (2,), True, False),
    (6, 2, 0, (3,), True, True),      # no Jacobian rows
]


@pytest.mark.parametrize('n,m,P,lead,a_var,b_var', SOLVE_CASES)
def test_solve(n, m, P, lead, a_var, b_var):
    from folx_amd import kernels as K

    print(f'case solve n={n} m={m} P={P} lead={lead} a_var={a_var} b_var={b_var}', flush=True)
    rng = np.random.default_rng(42)
    A = well_conditioned(rng, *lead, n=n)
    b = rand(rng, *lead, n, m)
    AJ = rand(rng, P, *lead, n, n) if a_var else None
    AL = rand(rng, *lead, n, n) if a_var else None
    bJ = rand(rng, P, *lead, n, m) if b_var else None
    bL = rand(rng, *lead, n, m) if b_var else None
    y, yJ, yL = rules.solve_rule(*f64(A, AJ, AL, b, bJ, bL))
    d = lambda a: None if a is None else dev(a)
    gy, gJ, gL = K.solve(dev(A), d(AJ), d(AL), dev(b), d(bJ), d(bL), P)
    close(gy, y, 'solution')
    if P:
        close(gJ, yJ, 'jacobian')
    close(gL, yL, 'laplacian', lap=True)


def _masks(rng, kind, n):
    if kind == 'rows':          # row i depends on the 3 coordinates of particle i
        return np.stack([np.broadcast_to((3 * np.arange(n) + t)[:, None], (n, n)) for t in range(3)])
    if kind == 'columns':
        return np.swapaxes(_masks(rng, 'rows', n), -1, -2).copy()
    if kind == 'two_rows':
        m = np.empty((6, n, n), np.int64)
        for i in range(n):
            deps = sorted([3 * i + t for t in range(3)] + [3 * ((i - 1) % n) + t for t in range(3)])
            m[:, i, :] = np.asarray(deps)[:, None]
        return m
    if kind == 'circulant':     # one entry per row and coordinate
        return np.stack([np.roll(np.arange(n), s) for s in range(n)])[None]
    m = rng.integers(-1, 2 * n, size=(2, n, n))  # ragged: holes, uneven widths
    m[1][m[1] == m[0]] = -1
    return m


@pytest.mark.parametrize('kind', ['rows', 'columns', 'two_rows', 'circulant', 'ragged'])
@pytest.mark.parametrize('n,lead', [(6, (5,)), (16, (3, 2)), (32, (2,)), (3, (4,))])
@pytest.mark.parametrize('variant', ['rows_of_A', 'entries', 'rows_of_At'])
def test_sparse_slogdet(kind, n, lead, variant):
    """All three table kinds on every mask; reference values = the dense slogdet rule on the
    materialised Jacobian."""
    from folx_amd import index_algebra as pia
    from folx_amd import kernels as K

    print(f'case sparse_slogdet {kind} n={n} lead={lead} {variant}', flush=True)
    rng = np.random.default_rng(43)
    mask = _masks(rng, kind, n)
    k = mask.shape[0]
    transposed = variant == 'rows_of_At'
    plan_mask = np.swapaxes(mask, -1, -2).copy() if transposed else mask
    cost, tables = pia.slogdet_factor_tables(plan_mask, variant == 'entries')
    C, rank, width = tables['take'].shape
    if rank > 64 or rank * width > 2048:
        pytest.skip('tables larger than the kernel holds in LDS')
    take, cols, rows = pia.slogdet_kernel_tables(tables, transposed, k, n)
    A = well_conditioned(rng, *lead, n=n)
    Jd = (rand(rng, k, *lead, n, n) * (mask >= 0).reshape(k, *([1] * len(lead)), n, n)).astype(np.float32)
    L = rand(rng, *lead, n, n)
    dense = oia.dense_array(Jd.astype(np.float64), np.broadcast_to(
        mask.reshape(k, *([1] * len(lead)), n, n), Jd.shape))
    sign, (ld, jac, lap) = rules.slogdet_rule(A.astype(np.float64), dense, L.astype(np.float64))
    gs, gld, gj, gl = K.sparse_slogdet(dev(A), dev(Jd), dev(L), dev(take, torch.int32), dev(cols, torch.int32),
                                       dev(rows, torch.int32), transposed)
    np.testing.assert_array_equal(gs.cpu().numpy(), sign)
    close(gld, ld, 'logdet')
    close(gj, jac[tables['coords']], 'jacobian')
    close(gl, lap, 'laplacian', lap=True)


# ---------------------------------------------------------------------------------------
# model level: the rules on the GPU against the dense oracle
# ---------------------------------------------------------------------------------------


def _run(fn, x, thr):
    """Strict bars of tests/tolerances.py, widened by the rounding noise that the matrices'
    conditioning puts on ANY fp32 evaluation: 4 x the distance between the numpy oracle run
    in float32 and in float64 (zero for well-conditioned inputs)."""
    import folx_amd
    from folx_amd import numpy as fnp
    from tolerances import LAP_ATOL, LAP_ATOL_REL, LAP_RTOL, VAL_ATOL_REL, VAL_RTOL

    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(torch.as_tensor(x).cuda())
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    r32 = fn(ob, ob.init_state(x, dtype=np.float32))
    J = out.jacobian.dense_array
    assert J.shape[0] <= ref.J.shape[0]
    assert not np.abs(ref.J[J.shape[0]:]).any()
    nJ = J.shape[0]

    def check(got, want, w32, rtol, atol_rel, atol, what):
        got = got.detach().cpu().numpy().astype(np.float64)
        floor = 4.0 * float(np.abs(np.asarray(w32, dtype=np.float64) - want).max())
        scale = float(np.abs(want).max())
        np.testing.assert_allclose(got, want, rtol=rtol, atol=atol + atol_rel * scale + floor, err_msg=what)

    check(out.x, ref.x, r32.x, VAL_RTOL, VAL_ATOL_REL, 0.0, 'x')
    check(J, ref.J[:nJ], r32.J[:nJ], VAL_RTOL, VAL_ATOL_REL, 0.0, 'jacobian')
    check(out.laplacian, ref.lap, r32.lap, LAP_RTOL, LAP_ATOL_REL, LAP_ATOL, 'laplacian')


@pytest.mark.parametrize('mode,batched', [('row_sparse', False), ('two_rows', False), ('columns', False),
                                          ('two_columns', False), ('shared_rows', False), ('row_sparse', True)])
@pytest.mark.parametrize('thr', [0, 18])
def test_slogdet_sparse_models(mode, batched, thr):
    from test_host_linalg import slater_model

    print(f'case slogdet model {mode} batched={batched} thr={thr}', flush=True)
    n = 6
    rng = np.random.default_rng(31)
    x = (0.4 * rng.normal(size=(3, n, 3))).astype(np.float32)
    w = rng.normal(size=(n, 3, n)).astype(np.float32)
    _run(slater_model(mode, w, batched), x, thr)


def _matrix(xp, x, W, n, lead=()):
    A = xp.reshape(xp.tanh(xp.dot(xp.reshape(x, (-1,)), W)), (*lead, n, n))
    return xp.add(A, n * np.eye(n, dtype=np.float32))


@pytest.mark.parametrize('thr', [0, 15])
def test_det_inv_solve_models(thr):
    print(f'case det/inv/solve models thr={thr}', flush=True)
    n = 5
    rng = np.random.default_rng(44)
    W = rng.normal(size=(3 * n, n * n)).astype(np.float32)
    Wb = rng.normal(size=(3 * n, 2 * n * n)).astype(np.float32)
    w = rng.normal(size=(n, 3, n)).astype(np.float32)
    A_const = (n * np.eye(n) + np.tril(rng.normal(size=(n, n)), -1)).astype(np.float32)
    b_mat = rng.normal(size=(n, 2)).astype(np.float32)
    x = rng.normal(size=(4, n, 3)).astype(np.float32)
    rhs = lambda xp, t: xp.sum(xp.tanh(t), axis=-1)

    def det_model(xp, t):
        A = xp.sum(xp.multiply(xp.expand_dims(t, -1), w), axis=1)
        return xp.det(xp.add(xp.tanh(A), n * np.eye(n, dtype=np.float32)))

    models = {
        'det': det_model,
        'inv': lambda xp, t: xp.inv(_matrix(xp, t, W, n)),
        'solve, matrix rhs': lambda xp, t: xp.solve(_matrix(xp, t, W, n), b_mat),
        'solve, both vary': lambda xp, t: xp.solve(_matrix(xp, t, W, n), rhs(xp, t)),
        'solve, rhs varies': lambda xp, t: xp.solve(A_const, rhs(xp, t)),
        'solve, batched matrix': lambda xp, t: xp.solve(_matrix(xp, t, Wb, n, lead=(2,)), rhs(xp, t)),
    }
    for name, fn in models.items():
        print('  model', name, flush=True)
        _run(fn, x, thr)

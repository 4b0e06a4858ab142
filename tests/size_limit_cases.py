"""Models at sizes beyond what the small-matrix kernels are built for (matrices larger than 32 x 32), shared by the
host-logic tests (CPU stand-ins) and the GPU tests.  The reference takes any size through jnp.linalg
(folx/slogdet.py:296-344, folx/linear_solve.py:54-145).  Every model maps a per-walker vector of 6 entries to its
output; the matrices are 34 x 34: a fixed well-conditioned matrix plus a low-rank part that depends on the input."""

import numpy as np

N_BIG = 34
_RNG = np.random.default_rng(91)
_BASE = (np.eye(N_BIG) * 2.5 + _RNG.normal(size=(N_BIG, N_BIG)) / np.sqrt(N_BIG)).astype(np.float32)
_U = (_RNG.normal(size=(6, N_BIG * N_BIG)) / N_BIG).astype(np.float32)
_RHS = _RNG.normal(size=(N_BIG, 3)).astype(np.float32)
_V = (_RNG.normal(size=(6, N_BIG)) / 2).astype(np.float32)


def _matrix(xp, x):
    """(34, 34) matrix whose every entry depends on all six inputs"""
    return xp.add(xp.reshape(xp.dot(xp.tanh(x), _U), (N_BIG, N_BIG)), _BASE)


BIG_MATRIX_FNS = {
    'slogdet': lambda xp, x: xp.slogdet(_matrix(xp, x))[1],
    'det': lambda xp, x: xp.multiply(xp.det(xp.multiply(_matrix(xp, x), 0.4)), 1.0),
    'inv': lambda xp, x: xp.sum(xp.tanh(xp.inv(_matrix(xp, x))), axis=0),
    'solve_const_rhs': lambda xp, x: xp.solve(_matrix(xp, x), _RHS),
    'solve_vector_rhs': lambda xp, x: xp.solve(_matrix(xp, x), xp.dot(xp.sin(x), _V)),
    'solve_const_matrix': lambda xp, x: xp.solve(_BASE, xp.reshape(xp.dot(xp.sin(x), _U[:, : N_BIG * 2]), (N_BIG, 2))),
}

"""Scatter models shared by the oracle, host-logic and GPU tests: the cases of the
reference's test/test_scatter.py written against the operator namespace ``xp``
(x has 12 entries; ``x.at[idx].op(u)`` becomes ``xp.scatter(x, idx, u, op)``)."""

import numpy as np

IDX = np.array([0, 2, 5])
DUP = np.array([1, 1, 3])
TRI = np.triu(np.ones((12, 12), dtype=np.float32))  # x @ TRI = cumsum(x)


def _g(xp, x, sl):
    return xp.getitem(x, (sl,))


def _dist(xp, x):
    r = xp.reshape(x, (-1, 3))
    return xp.sqrt(xp.sum(xp.square(r), axis=1))


def rows_into_zeros(xp, x):  # test_scatter.py:36-43 (issue #28 pattern)
    d = _dist(xp, x)
    sph = xp.scatter(np.zeros((2, 4), dtype=np.float32), 0, d, 'set')
    return xp.scatter(sph, 1, xp.multiply(d, 5.0), 'set')


def multi_dim_indices(xp, x):  # test_scatter.py:72-75
    r = xp.reshape(xp.sin(x), (4, 3))
    i, j = np.array([0, 3, 0]), np.array([1, 2, 1])
    return xp.scatter(r, (i, j), xp.multiply(_g(xp, x, slice(0, 3)), _g(xp, x, slice(3, 6))), 'add')


CASES = {
    # set (test_scatter.py:32-56)
    'rows_into_zeros': rows_into_zeros,
    'fancy_set': lambda xp, x: xp.scatter(xp.sin(x), IDX, xp.multiply(_g(xp, x, slice(0, 3)), 2.0), 'set'),
    'const_updates_set': lambda xp, x: xp.scatter(xp.sin(x), IDX, 1.5, 'set'),
    'scalar_index': lambda xp, x: xp.scatter(
        xp.sin(x), 3, xp.multiply(xp.getitem(x, (0,)), xp.getitem(x, (1,))), 'set'),
    # add (test_scatter.py:58-83)
    'segment_sum': lambda xp, x: xp.scatter(np.zeros((2,), dtype=np.float32), np.array([0, 1, 0, 1]),
                                            _dist(xp, x), 'add'),
    'duplicate_add': lambda xp, x: xp.scatter(xp.sin(x), DUP, xp.square(_g(xp, x, slice(0, 3))), 'add'),
    'windowed_add': lambda xp, x: xp.scatter(
        xp.reshape(xp.sin(x), (4, 3)), np.array([0, 2]),
        xp.reshape(xp.cos(_g(xp, x, slice(0, 6))), (2, 3)), 'add'),
    'multi_dim_indices': multi_dim_indices,
    'const_updates_add': lambda xp, x: xp.scatter(xp.sin(x), DUP, 2.5, 'add'),
    # min / max (test_scatter.py:85-94)
    'min': lambda xp, x: xp.scatter(xp.sin(x), IDX, xp.multiply(_g(xp, x, slice(6, 9)), 2.0), 'min'),
    'max': lambda xp, x: xp.scatter(xp.sin(x), IDX, xp.multiply(_g(xp, x, slice(6, 9)), 2.0), 'max'),
    'min_const': lambda xp, x: xp.scatter(xp.sin(x), IDX, 0.1, 'min'),
    'max_const': lambda xp, x: xp.scatter(xp.sin(x), IDX, -0.1, 'max'),
    'min_duplicates': lambda xp, x: xp.scatter(xp.sin(x), DUP, _g(xp, x, slice(6, 9)), 'min'),
    # dynamic_update_slice (test_scatter.py:125-137)
    'dus': lambda xp, x: xp.scatter(xp.sin(x), slice(4, 7), xp.multiply(_g(xp, x, slice(0, 3)), 2.0), 'set'),
    'dus_const': lambda xp, x: xp.scatter(xp.sin(x), slice(4, 7), np.ones(3, dtype=np.float32), 'set'),
}

# one argument dense at threshold 4 (cumsum), the other sparse (test_scatter.py:96-123)
MIXED = {
    'dense_op_set': lambda xp, x: xp.scatter(xp.dot(x, TRI), IDX, xp.multiply(_g(xp, x, slice(0, 3)), 2.0), 'set'),
    'dense_upd_set': lambda xp, x: xp.scatter(xp.sin(x), IDX, _g(xp, xp.dot(x, TRI), slice(0, 3)), 'set'),
    'dense_op_add': lambda xp, x: xp.scatter(xp.dot(x, TRI), IDX, xp.multiply(_g(xp, x, slice(0, 3)), 2.0), 'add'),
    'dense_upd_add': lambda xp, x: xp.scatter(xp.sin(x), IDX, _g(xp, xp.dot(x, TRI), slice(0, 3)), 'add'),
    'dense_upd_min': lambda xp, x: xp.scatter(xp.sin(x), IDX, _g(xp, xp.dot(x, TRI), slice(0, 3)), 'min'),
}


def min_max_elementwise(xp, x):
    a, b = xp.sin(_g(xp, x, slice(0, 6))), xp.cos(_g(xp, x, slice(6, 12)))
    return xp.add(xp.minimum(a, b), xp.maximum(xp.multiply(a, 2.0), 0.3))


def fancy_take(xp, x):
    """Integer-array indexing (the ``gather`` primitive): a circulant built from one take."""
    n = 6
    perm = np.stack([np.roll(np.arange(n), s) for s in range(n)])
    t = xp.tanh(xp.getitem(x, (slice(0, n),)))
    A = xp.getitem(t, (perm,))                              # (n, n)
    picked = xp.getitem(xp.reshape(xp.sin(x), (4, 3)), (np.array([3, 0, 0]), np.array([1, 2, -1])))
    return xp.add(xp.sum(xp.multiply(A, A), axis=1), xp.sum(picked))

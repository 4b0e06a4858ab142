"""Pins the oracle's scatter and min / max rules by brute-force AD (the cases of the
reference's test/test_scatter.py) and its scatter mask algebra by hand-derived cases."""

import numpy as np
import pytest

from bruteforce import brute_force, plain
from oracle import backend as ob
from oracle import index_algebra as ia
import composed_cases
from scatter_cases import CASES, MIXED, fancy_take, min_max_elementwise


def _check(fn, x):
    out = fn(ob, ob.init_state(x, dtype=np.float64))
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x)
    np.testing.assert_allclose(out.x, by, rtol=2e-5, atol=1e-9)
    np.testing.assert_allclose(out.J, bJ, rtol=2e-5, atol=1e-9)
    np.testing.assert_allclose(out.lap, bL, rtol=2e-5, atol=1e-8)


@pytest.mark.parametrize('name', sorted(CASES) + sorted(MIXED))
def test_scatter_vs_bruteforce(name):
    fn = CASES.get(name) or MIXED[name]
    _check(fn, np.random.default_rng(50).normal(size=(2, 12)))


@pytest.mark.parametrize('name', sorted(composed_cases.CASES))
def test_composed_rules_vs_bruteforce(name):
    _check(composed_cases.CASES[name], np.random.default_rng(53).normal(size=(2, 12)))


def test_min_max_vs_bruteforce():
    _check(min_max_elementwise, np.random.default_rng(51).normal(size=(3, 12)))


def test_integer_array_indexing_vs_bruteforce():
    _check(fancy_take, np.random.default_rng(52).normal(size=(2, 12)))


def test_scatter_out_mask_hand_cases():
    # operand sin(x): position p depends on input p; updates x[:3] * 2 land on 0, 2, 5
    op = np.arange(6)[None]
    upd = np.arange(3)[None]
    tpos = np.array([0, 2, 5])
    got = ia.scatter_out_mask(op, upd, tpos, (6,), is_set=True)
    np.testing.assert_array_equal(got, [[0, 1, 1, 3, 4, 2]])           # overwritten: updates only
    got = ia.scatter_out_mask(op, upd, tpos, (6,), is_set=False)
    np.testing.assert_array_equal(got, [[0, 1, 1, 3, 4, 2], [-1, -1, 2, -1, -1, 5]])  # union, ascending
    # duplicates and a dropped update; constant operand
    got = ia.scatter_out_mask(None, np.array([[4, 7, 5, 9]]), np.array([1, 1, -1, 0]), (2,), is_set=False)
    np.testing.assert_array_equal(got, [[9, 4], [-1, 7]])
    # nothing depends on anything: one row of -1
    got = ia.scatter_out_mask(None, np.array([[-1, -1]]), np.array([0, 1]), (3,), is_set=True)
    np.testing.assert_array_equal(got, [[-1, -1, -1]])

"""Host index algebra of the product (vectorised numpy) against the oracle's explicit
loops on random masks, and against the reference's exact-integer find_out_idx cases."""

import numpy as np
import pytest

from folx_amd import index_algebra as pa
from oracle import index_algebra as oa
from test_oracle_index import CASES, run_case


@pytest.mark.parametrize('c', CASES, ids=[c['name'] for c in CASES])
def test_find_out_idx_golden(c):
    def fo(masks, x_shapes, in_axes, lio, thr):
        masks = [None if m is None else m for m in masks]
        return pa.find_out_idx(masks, x_shapes, in_axes, lio, thr)

    run_case(fo, oa.dense_mask, c)


def random_mask(rng, k, shape, n_in=9, p_invalid=0.25):
    m = rng.integers(0, n_in, size=(k, *shape))
    m[rng.random(m.shape) < p_invalid] = -1
    return m


@pytest.mark.parametrize('seed', range(6))
def test_find_out_idx_random(seed):
    rng = np.random.default_rng(seed)
    shapes = [((3, 4), (3, 4)), ((3, 1), (1, 4)), ((2, 3, 2), (3, 1)), ((4,), (4,))][seed % 4]
    masks = [random_mask(rng, int(rng.integers(1, 4)), s) for s in shapes]
    for lio in (False, True):
        got = pa.find_out_idx(masks, [list(s) for s in shapes], [(), ()], lio, 5)
        ref = oa.find_out_idx(masks, [list(s) for s in shapes], [(), ()], lio, 5)
        assert got[1] == ref[1]
        np.testing.assert_array_equal(got[0], ref[0])
    # with consumed axes
    m = random_mask(rng, 2, (3, 4))
    got = pa.find_out_idx([m], [[3, 4]], [(1,)], False, 50)
    ref = oa.find_out_idx([m], [[3, 4]], [(1,)], False, 50)
    np.testing.assert_array_equal(got[0], ref[0])


@pytest.mark.parametrize('seed', range(4))
def test_gather_table_matches_materialize(seed):
    rng = np.random.default_rng(seed)
    k, shape, n_out = 4, (3, 5), 6
    idx = rng.integers(-1, n_out, size=(k, *shape))
    data = rng.normal(size=(k, 2, *shape))
    take = pa.gather_table(idx, n_out)
    assert take.shape[0] == n_out and take.shape[2:] == shape
    out = np.zeros((n_out, 2, *shape))
    for t in range(n_out):
        for s in range(take.shape[1]):
            src = take[t, s]
            for pos in np.ndindex(*shape):
                if src[pos] >= 0:
                    out[(t, slice(None), *pos)] += data[(src[pos], slice(None), *pos)]
    np.testing.assert_allclose(out, oa.materialize(data, idx, n_out))
    # sources keep their order within a target
    for pos in np.ndindex(*shape):
        for t in range(n_out):
            col = [int(v) for v in take[(t, slice(None), *pos)] if v >= 0]
            assert col == sorted(col)


@pytest.mark.parametrize('seed', range(4))
def test_get_index_mask(seed):
    rng = np.random.default_rng(seed)
    mask = random_mask(rng, 3, (4, 2))
    outputs = random_mask(rng, 5, (4, 1))
    np.testing.assert_array_equal(pa.get_index_mask(mask, outputs), oa.get_index_mask(mask, outputs))
    outputs = np.arange(9)[:, None, None]
    np.testing.assert_array_equal(pa.get_index_mask(mask, outputs), oa.get_index_mask(mask, outputs))


@pytest.mark.parametrize('seed', range(4))
def test_reduction_frame_and_sum_out_mask(seed):
    rng = np.random.default_rng(seed)
    m1 = random_mask(rng, 2, (3, 4, 2))
    m2 = random_mask(rng, 1, (3, 1, 2))
    for axes in [(1,), (0, 2), (2,), (0, 1, 2)]:
        np.testing.assert_array_equal(pa.reduction_frame([m1, m2], axes), oa.reduction_frame([m1, m2], axes))
        got, slot = pa.sum_out_mask(m1, axes)
        ref, rslot = oa.sum_out_mask(m1, axes)
        np.testing.assert_array_equal(got, ref)
        np.testing.assert_array_equal(slot, rslot)


def test_merge_rows_and_duplicates():
    rng = np.random.default_rng(0)
    a, b = random_mask(rng, 2, (3, 2)), random_mask(rng, 3, (3, 1))
    b[1] = np.broadcast_to(a[0][:, :1], (3, 1))
    res, inv = pa.merge_rows([a, b])
    rres, rinv = oa.merge_binary_masks([a, b])
    np.testing.assert_array_equal(res, rres)
    np.testing.assert_array_equal(inv, rinv)
    for m in (a, b, np.array([[1, 2], [1, 3]]), np.array([[-1, 2], [-1, 3]])):
        assert pa.has_duplicates(m) == oa.has_duplicates(m)


def test_dot_projection_and_split_inner():
    for thr in (3, 4):
        got = pa.dot_projection(oa.init_mask((6, 4)), -1, thr)
        ref = oa.dot_projection(oa.init_mask((6, 4)), -1, thr)
        assert (got[0] is None) == (ref[0] is None) and got[1] == ref[1]
        if got[0] is not None:
            np.testing.assert_array_equal(got[0], ref[0])
    node = np.broadcast_to(np.arange(5)[None, :, None], (2, 5, 7))
    assert pa.split_inner(node) == 1
    assert pa.split_inner(np.arange(10).reshape(1, 5, 2)) == 0
    assert pa.split_inner(np.zeros((3, 4, 5), dtype=int)) == 2

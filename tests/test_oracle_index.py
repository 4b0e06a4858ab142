"""Pins oracle.index_algebra: the 14 exact-integer cases of the reference's
test/test_find_out_idx.py (committed as data in tests/golden/find_out_idx_cases.json), and
set-enumeration checks for the remaining index functions."""

import json
import os

import numpy as np
import pytest

from oracle import index_algebra as ia

HERE = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(HERE, 'golden', 'find_out_idx_cases.json')) as f:
    CASES = json.load(f)


def run_case(find_out_idx, dense_mask, c):
    masks = []
    for m, xs in zip(c['masks'], c['x_shapes']):
        masks.append(None if m is None else np.asarray(m, dtype=np.int32))
    if c['expect_none']:
        out, dense = find_out_idx(masks, c['x_shapes'], [tuple(a) for a in c['in_axes']],
                                  c['linear_in_one'], c['threshold'])
        assert out is None and dense is True
        return
    out, dense = find_out_idx(masks, c['x_shapes'], [tuple(a) for a in c['in_axes']],
                              c['linear_in_one'], c['threshold'])
    assert dense is c['dense'], c['name']
    if c['idx'] is not None:
        exp = np.asarray(c['idx'], dtype=np.int64)
        assert out.shape == exp.shape, c['name']
        np.testing.assert_array_equal(out, exp)
    if c['shape'] is not None:
        for got, want in zip(out.shape, c['shape']):
            assert want is None or got == want, (c['name'], out.shape)
        assert len(out.shape) == len(c['shape'])
    if c['columns'] is not None:
        for key, want in c['columns'].items():
            pos = tuple(int(v) for v in key.split(','))
            col = sorted(int(v) for v in out[(slice(None), *pos)] if v >= 0)
            assert col == want, (c['name'], key, col)


@pytest.mark.parametrize('c', CASES, ids=[c['name'] for c in CASES])
def test_find_out_idx_golden(c):
    run_case(ia.find_out_idx, ia.dense_mask, c)


def test_materialize_and_dense_array():
    rng = np.random.default_rng(0)
    mask = np.array([[[0, 3], [2, 2]], [[1, -1], [2, 5]]])  # (k=2, 2, 2); duplicate 2 at (1,0)
    data = rng.normal(size=(2, 3, 2, 2))  # (k, B, 2, 2)
    dense = ia.dense_array(data, mask)
    assert dense.shape == (6, 3, 2, 2)
    np.testing.assert_allclose(dense[0, :, 0, 0], data[0, :, 0, 0])
    np.testing.assert_allclose(dense[1, :, 0, 0], data[1, :, 0, 0])
    np.testing.assert_allclose(dense[3, :, 0, 1], data[0, :, 0, 1])
    np.testing.assert_allclose(dense[2, :, 1, 0], data[0, :, 1, 0] + data[1, :, 1, 0])
    np.testing.assert_allclose(dense[5, :, 1, 1], data[1, :, 1, 1])
    assert np.count_nonzero(dense) == 3 * 6
    assert ia.has_duplicates(mask) and not ia.has_duplicates(mask[:1])


def test_get_index_mask_first_match():
    mask = np.array([[4, 7], [9, -1]])
    outputs = np.array([[7, 7], [4, 9], [9, -1]])
    got = ia.get_index_mask(mask, outputs)
    np.testing.assert_array_equal(got, [[1, 0], [2, 2]])  # -1 matches a -1 slot (api.py:136-141)
    got = ia.get_index_mask(mask, np.arange(10)[:, None])
    np.testing.assert_array_equal(got, [[4, 7], [9, -1]])


def test_reduction_frame_pads_at_end():
    # one row, node-wise features: reducing the feature axis unions 4 inputs per node
    mask = ia.init_mask((3, 4))
    fr = ia.reduction_frame([mask], (1,))
    np.testing.assert_array_equal(fr, np.arange(12).reshape(3, 4).T)
    m = np.array([[[0, -1, 2], [5, 5, -1]]])
    np.testing.assert_array_equal(ia.reduction_frame([m], (1,)), [[0, 5], [2, -1]])


def test_sum_out_mask_minus_one_sorts_first():
    m = np.array([[[0, -1, 2], [5, 5, 5]]])  # (1, 2, 3) reduce last axis
    idx_out, slot = ia.sum_out_mask(m, (1,))
    np.testing.assert_array_equal(idx_out, [[-1, 5], [0, -1], [2, -1]])
    np.testing.assert_array_equal(slot, [[[1, 0, 2], [0, 0, 0]]])


def test_merge_binary_masks_unique_rows():
    a = np.array([[3, 4, 5]])
    b = np.array([[0, 0, 0], [3, 4, 5]])
    res, inv = ia.merge_binary_masks([a, b])
    np.testing.assert_array_equal(res, [[0, 0, 0], [3, 4, 5]])
    np.testing.assert_array_equal(inv, [1, 0, 1])


def test_add_masks():
    a = np.array([[1, 2]])
    assert ia.add_masks(a, a.copy())[0] == 'same'
    kind, m = ia.add_masks(a, np.array([[1, 3]]))
    assert kind == 'concat' and m.shape == (2, 2)


def test_dot_projection():
    # mask constant along the contracted axis: rows pass through (k stays 1)
    node = np.broadcast_to(np.arange(5)[None, :, None], (1, 5, 7))
    proj, aligned = ia.dot_projection(node, -1, threshold=4)
    assert not aligned and proj.shape == (1, 5, 1)
    # the README sparse case: (1, 100, 4) initial mask, contract features -> k = 4
    proj, aligned = ia.dot_projection(ia.init_mask((6, 4)), -1, threshold=4)
    assert aligned and proj.shape == (4, 6, 1)
    np.testing.assert_array_equal(proj[:, 2, 0], [8, 9, 10, 11])
    assert ia.dot_projection(ia.init_mask((6, 4)), -1, threshold=3)[0] is None

"""Writes find_out_idx_cases.json: the exact-integer known-answer cases of the reference's
test/test_find_out_idx.py, transcribed by hand as data (inputs and expected outputs).

Each case: masks (int lists, null = dense Jacobian with 3 rows), x_shapes, in_axes,
linear_in_one (True = FunctionFlags.LINEAR_IN_ONE, False = GENERAL), threshold, and the
expectation: ``idx`` (full array), or ``shape`` / ``columns`` (partial checks the reference
makes), plus ``dense``.  Line numbers refer to test/test_find_out_idx.py.
"""

import json
import os

import numpy as np

cases = []


def case(name, line, masks, in_axes, lio, thr, dense, x_shapes=None, idx=None, shape=None, columns=None, none=False):
    if x_shapes is None:
        x_shapes = [list(np.asarray(m).shape[1:]) for m in masks]
    cases.append(
        dict(name=name, ref_line=line, masks=masks, x_shapes=x_shapes, in_axes=in_axes,
             linear_in_one=lio, threshold=thr, dense=dense, idx=idx, shape=shape,
             columns=columns, expect_none=none)
    )


m1 = [[0, 1, 2], [3, 4, -1]]
m2 = [[0, 1, 5], [6, 4, -1]]
case('no_weak_jac_returns_none_dense', 58, [None], [[]], False, 10, True, x_shapes=[[4]], none=True)
case('single_jac_already_unique', 65, [m1], [[]], False, 100, False, idx=[[0, 1, 2], [3, 4, -1]])
case('two_jacs_union', 73, [m1, m2], [[], []], False, 100, False,
     idx=[[0, 1, 2], [3, 4, 5], [6, -1, -1]])
case('two_jacs_intersect', 86, [m1, m2], [[], []], True, 100, False,
     idx=[[0, 1, -1], [-1, 4, -1]])
m3 = [[[0, 1, 2], [10, 11, 12]], [[3, 4, -1], [13, 14, -1]]]
case('extra_broadcast_dim', 101, [m3], [[]], False, 100, False, idx=m3, shape=[2, 2, 3])
case('broadcast_with_size_one_axis', 113,
     [[[[0], [1], [2]], [[3], [4], [-1]]], [[[5, 6, 7]], [[-1, 8, 9]]]],
     [[], []], False, 100, False, shape=[None, 3, 3],
     columns={'0,0': [0, 3, 5], '2,2': [2, 7, 9]})
case('threshold_triggers_dense', 132, [[[0, 1], [2, 3]]], [[]], False, 1, True, shape=[2, 2])
case('dense_when_at_max_size', 142,
     [[[0, 0, 0, 0], [1, 1, 1, 1], [2, 2, 2, 2], [3, 3, 3, 3]]], [[]], False, 100, True,
     shape=[4, 4])
case('all_invalid_mask', 156, [[[-1, -1, -1], [-1, -1, -1]]], [[]], False, 100, True, shape=[0, 3])
case('duplicate_indices_same_column', 166, [[[0, 1, 2], [0, 1, 2]]], [[]], False, 100, False,
     idx=[[0, 1, 2]])
case('with_vmap_axes', 175, [np.arange(24).reshape(2, 4, 3).tolist()], [[0]], False, 100, False,
     x_shapes=[[4, 3]], shape=[8, 3], columns={'0': [0, 3, 6, 9, 12, 15, 18, 21]})
case('three_jacs_union', 192,
     [[[0, 1], [2, -1]], [[1, 3], [4, -1]], [[5, 1], [-1, -1]]], [[], [], []], False, 100, True,
     idx=[[0, 1], [1, 3], [2, -1], [4, -1], [5, -1]])
case('three_jacs_intersect', 208,
     [[[0, 1], [2, -1]], [[1, 3], [0, -1]], [[5, 1], [0, -1]]], [[], [], []], True, 100, False,
     idx=[[0, -1]])
case('two_jacs_different_K', 224,
     [[[0, 1], [2, 3]], [[10, 11], [12, 13], [-1, -1]]], [[], []], False, 100, True,
     idx=[[0, 1], [2, 3], [10, 11], [12, 13]])

with open(os.path.join(os.path.dirname(__file__), 'find_out_idx_cases.json'), 'w') as f:
    json.dump(cases, f, indent=1)
print(len(cases), 'cases written')

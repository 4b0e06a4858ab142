"""Models with ONE derivative-carrying operand multiplied with a constant of any rank, on either side,
under any contracted and batch axes: the forms ``_dot_general_one_constant`` of the reference takes
(folx/wrapped_functions.py:71-171).  Shared by the host-logic tests (CPU stand-ins) and the GPU tests.
Every model maps a per-walker array of shape (4, 3) to its output."""

import numpy as np

_RNG_W = np.random.default_rng(77)
_W_HEADS = _RNG_W.normal(size=(4, 3, 5)).astype(np.float32) / 2      # per-"head" weights: batch axis of size 4
_W_VEC = _RNG_W.normal(size=(3,)).astype(np.float32)
_W_LEFT3 = _RNG_W.normal(size=(4, 6, 3)).astype(np.float32) / 2
_W_BIG = _RNG_W.normal(size=(2, 6, 7)).astype(np.float32) / 3
_W_NHD = _RNG_W.normal(size=(3, 2, 2)).astype(np.float32) / 2      # (H, d, e) for h (n, H, d) = (4, 3) -> (2, 3, 2)
ONE_CONSTANT_FNS = {
    # per-head weights on an (n, H, d) activation, as einsum and as matmul
    'nhd_hde': lambda xp, x: xp.einsum('nhd,hde->nhe', xp.reshape(xp.tanh(x), (2, 3, 2)), _W_NHD),
    'nhd_matmul': lambda xp, x: xp.matmul(xp.reshape(xp.tanh(x), (2, 3, 1, 2)), _W_NHD),    # (2,3,1,2)@(3,2,2)
    'W_matmul_h': lambda xp, x: xp.matmul(np.arange(20.0, dtype=np.float32).reshape(5, 4) / 20, xp.sin(x)),  # (5,4)@(4,3)
    # a constant operand with batch axes (folx/wrapped_functions.py:71-171 takes any dimension numbers)
    'einsum_heads': lambda xp, x: xp.einsum('nd,nde->ne', xp.tanh(x), _W_HEADS),               # batch n, (4,3)x(4,3,5)
    'einsum_heads_T': lambda xp, x: xp.einsum('nde,nd->en', _W_HEADS, xp.tanh(x)),             # constant on the left
    'matmul_w3d': lambda xp, x: xp.matmul(xp.expand_dims(xp.sin(x), 1), _W_HEADS),             # (4,1,3)@(4,3,5)
    'matmul_w3d_bcast': lambda xp, x: xp.matmul(xp.sin(x), _W_HEADS),                          # (4,3)@(4,3,5) -> (4,4,5)
    'matmul_left3d': lambda xp, x: xp.matmul(_W_LEFT3, xp.expand_dims(xp.cos(x), 2)),          # (4,6,3)@(4,3,1)
    'matmul_vec': lambda xp, x: xp.matmul(xp.tanh(x), _W_VEC),                                 # (4,3)@(3,) -> (4,)
    'vec_matmul': lambda xp, x: xp.matmul(np.arange(4.0, dtype=np.float32) / 4, xp.tanh(x)),   # (4,)@(4,3) -> (3,)
    # contraction over a non-last axis of the operand with derivatives, and over two axes at once
    'contract_first': lambda xp, x: xp.dot_general(xp.tanh(x), np.arange(8.0, dtype=np.float32).reshape(4, 2) / 8,
                                                   (((0,), (0,)), ((), ()))),                   # -> (3, 2)
    'contract_two': lambda xp, x: xp.dot_general(_W_BIG, xp.reshape(xp.sin(x), (2, 6)),
                                                 (((0, 1), (0, 1)), ((), ()))),                 # -> (7,)
    'batch_and_free': lambda xp, x: xp.dot_general(xp.reshape(xp.tanh(x), (2, 2, 3)), _W_BIG[:, :3, :],
                                                   (((2,), (1,)), ((0,), (0,)))),               # -> (2, 2, 7)
}

"""folx_amd -- forward-Laplacian propagation on AMD MI355X (gfx950).

Public surface (same names as microsoft/folx, folx/__init__.py:14-25):
``forward_laplacian``, ``ForwardLaplacianOperator``, ``FwdLaplArray``, ``FwdJacobian``,
``register_function`` / ``deregister_function``, ``batched_vmap``; plus ``vmap`` (the
walker axis is part of the data layout), ``jit`` (HIP-graph replay) and ``folx_amd.numpy`` (the functions a model is
written with).  All arithmetic runs in ``libfolx_hip.so``; there is no CPU path.
"""

from .api import BatchedArray, FunctionFlags, FwdJacobian, FwdLaplArray
from .graph import jit
from .interpreter import forward_laplacian, init_forward_laplacian_state
from .operators import ForwardLaplacianOperator, LoopLaplacianOperator, ParallelLaplacianOperator
from .vmap import batched_vmap, vmap
from .wrapped_functions import deregister_function, get_laplacian, is_registered, register_function

__all__ = [
    'BatchedArray',
    'FunctionFlags',
    'FwdJacobian',
    'FwdLaplArray',
    'ForwardLaplacianOperator',
    'batched_vmap',
    'deregister_function',
    'LoopLaplacianOperator',
    'ParallelLaplacianOperator',
    'forward_laplacian',
    'get_laplacian',
    'init_forward_laplacian_state',
    'is_registered',
    'jit',
    'register_function',
    'vmap',
]

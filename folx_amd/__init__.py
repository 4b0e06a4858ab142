"""folx_amd -- forward-Laplacian propagation on AMD MI355X (gfx950).

Public surface (same names as microsoft/folx, folx/__init__.py:14-25):
``forward_laplacian``, ``ForwardLaplacianOperator``, ``FwdLaplArray``, ``FwdJacobian``,
``register_function`` / ``deregister_function``, ``wrap_forward_laplacian``, ``warp_without_fwd_laplacian``,
``batched_vmap``; plus ``vmap`` (the
walker axis is part of the data layout), ``jit`` (HIP-graph replay) and ``folx_amd.numpy`` (the functions a model is
written with).  All arithmetic of the registered rules runs in ``libfolx_hip.so``; there is no CPU path.  (The
generic rule that ``wrap_forward_laplacian`` builds for a caller's own torch function differentiates that function
with ``torch.func``, since nothing else defines its derivatives.)
"""

from .api import BatchedArray, FunctionFlags, FwdJacobian, FwdLaplArray
from .graph import jit
from .interpreter import forward_laplacian, init_forward_laplacian_state
from .fx import forward_laplacian_torch
from .operators import (
    ForwardLaplacianOperator,
    Laplacian,
    LaplacianOperator,
    LoopLaplacianOperator,
    ParallelLaplacianOperator,
)
from .vmap import batched_vmap, vmap
from .wrapped_functions import deregister_function, get_laplacian, is_registered, register_function
from .wrapper import custom_jvp, warp_without_fwd_laplacian, wrap_elementwise, wrap_forward_laplacian

__all__ = [
    'BatchedArray',
    'FunctionFlags',
    'FwdJacobian',
    'FwdLaplArray',
    'ForwardLaplacianOperator',
    'batched_vmap',
    'deregister_function',
    'Laplacian',
    'LaplacianOperator',
    'LoopLaplacianOperator',
    'ParallelLaplacianOperator',
    'forward_laplacian',
    'get_laplacian',
    'init_forward_laplacian_state',
    'is_registered',
    'jit',
    'register_function',
    'vmap',
    'warp_without_fwd_laplacian',
    'wrap_elementwise',
    'wrap_forward_laplacian',
    'custom_jvp',
    'forward_laplacian_torch',
]

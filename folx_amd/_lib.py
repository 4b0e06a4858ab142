"""ctypes binding of ``libfolx_hip.so`` -- the only way the package reaches the GPU kernels.

The library must have been built (``python -m folx_amd.build``); there is no fallback:
``load()`` raises when it is missing or lacks a symbol.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBPATH = os.path.join(_HERE, 'lib', 'libfolx_hip.so')

OK, EINVAL, ENOTSUP, ELAUNCH, ESCRATCH = 0, -1, -2, -3, -4
STATIC_SCRATCH_BYTES = 64 << 20

# name -> (restype, argtypes); mirrors include/folx_hip.h one to one
_P = c_void_p
SIGNATURES = {
    'folx_hip_version': (c_int, []),
    'folx_hip_strerror': (c_char_p, [c_int]),
    'folx_hip_set_gemm_mode': (c_int, [c_int]),
    'folx_hip_get_gemm_mode': (c_int, []),
    'folx_hip_dense_fwdlap': (c_int, [_P] * 12 + [c_int64, c_int32, c_int32, c_int32]),
    'folx_hip_dense_rows_fwdlap': (c_int, [_P] * 12 + [c_int64, c_int32, c_int32, c_int32, c_int64, c_int64]),
    'folx_hip_dense_act_workspace_bytes': (c_int64, [c_int64, c_int32, c_int32, c_int32]),
    'folx_hip_dense_act_fwdlap': (c_int, [_P, c_int32, c_float] + [_P] * 11 + [c_int64, c_int32, c_int32, c_int32, _P, c_int64]),
    'folx_hip_dense_act_parts_fwdlap': (c_int, [_P, c_int32, c_float, _P, _P, c_int32, _P, _P, _P, c_int32] + [_P] * 11
                                        + [c_int64, c_int32, c_int32, _P, c_int64]),
    'folx_hip_norm_dense_workspace_bytes': (c_int64, [c_int64, c_int32, c_int32, c_int32, c_int32]),
    'folx_hip_norm_dense_fwdlap': (c_int, [_P, c_int32, c_float] + [_P] * 5 + [c_float] + [_P] * 5
                                   + [c_int64, c_int32, c_int32, c_int32, _P, c_int64]),
    'folx_hip_norm_dense_static_fwdlap': (c_int, [_P, c_int32, c_float] + [_P] * 5 + [c_float] + [_P] * 5
                                          + [c_int64, c_int32, c_int32, c_int32]),
    'folx_hip_dot_two_fwdlap': (c_int, [_P] * 10 + [c_int64, c_int32, c_int32, c_int32, c_int32, c_int32, _P]),
    'folx_hip_layernorm_fwdlap': (c_int, [_P] * 9 + [c_int64, c_int32, c_int32, c_float]),
    'folx_hip_elementwise_fwdlap': (c_int, [_P, c_int32, c_float, _P, _P, _P, _P, _P, _P, c_int64, c_int32]),
    'folx_hip_exp_envelope_fwdlap': (c_int, [_P] * 9 + [c_int64, c_int32, c_int32, c_int32]),
    'folx_hip_binary_fwdlap': (c_int, [_P, c_int32, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int64, c_int32]),
    'folx_hip_mul_sparse_fwdlap': (c_int, [_P] * 11 + [c_int64, c_int64, c_int32, c_int32]),
    'folx_hip_rows_affine': (c_int, [_P, _P, _P, c_int64, c_int64, _P, _P, c_float, c_float, _P]),
    'folx_hip_reduce_sum': (c_int, [_P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_float]),
    'folx_hip_reduce_sum_window': (c_int, [_P, _P, _P, c_int64, c_int64, c_int64, c_int64, c_int64, c_int64, c_float]),
    'folx_hip_reduce_max': (c_int, [_P, _P, _P, c_int64, c_int64, c_int64]),
    'folx_hip_gather_rows': (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int32, c_int64, c_int64, c_int64]),
    'folx_hip_gather_reduce_rows': (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int32, c_int64, c_int64, c_int32, c_int64,
                                            c_int64, c_float]),
    'folx_hip_gather_cols': (c_int, [_P, _P, _P, _P, c_int64, c_int64, c_int64, c_int32, c_int64]),
    'folx_hip_scatter_add_rows': (c_int, [_P, _P, _P, _P, c_int32, c_int32, c_int64, c_int64, c_int64]),
    'folx_hip_slogdet_fwdlap': (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int32, c_int32]),
    'folx_hip_slogdet_strided_fwdlap': (c_int, [_P] * 8 + [c_int64, c_int64, c_int32, c_int32] + [c_int64] * 4),
    'folx_hip_slogdet_scaled_fwdlap': (c_int, [_P] * 12 + [c_int64, c_int64, c_int32, c_int32] + [c_int64] * 5 + [c_int32]),
    'folx_hip_sparse_slogdet_fwdlap': (c_int, [_P] * 11 + [c_int64] + [c_int32] * 6),
    'folx_hip_inv_fwdlap': (c_int, [_P] * 7 + [c_int64, c_int32, c_int32]),
    'folx_hip_inv_values': (c_int, [_P] * 5 + [c_int64, c_int32]),
    'folx_hip_trace_pair': (c_int, [_P] * 4 + [c_int64, c_int32]),
    'folx_hip_solve_fwdlap': (c_int, [_P] * 10 + [c_int64, c_int32, c_int32, c_int32]),
    'folx_hip_mhsa_fwdlap': (c_int, [_P] * 15 + [c_int64, c_int32, c_int32, c_int32, c_int32]),
    'folx_hip_mhsa_sparse_fwdlap': (c_int, [_P] * 14 + [c_int64, c_int32, c_int32, c_int32, c_int32]),
    'folx_hip_mhsea_fwdlap': (c_int, [_P] * 18 + [c_int64, c_int32, c_int32, c_int32, c_int32]),
}

ACT = {
    'tanh': 0, 'silu': 1, 'exp': 2, 'log': 3, 'sqrt': 4, 'rsqrt': 5, 'square': 6,
    'logistic': 7, 'sigmoid': 7, 'softplus': 8, 'sin': 9, 'cos': 10, 'abs': 11,
    'log1p': 12, 'reciprocal': 13, 'expm1': 14, 'integer_pow': 15,
    'sinh': 16, 'cosh': 17, 'tan': 18, 'asin': 19, 'acos': 20, 'atan': 21, 'asinh': 22, 'acosh': 23,
    'atanh': 24, 'erf': 25, 'erfc': 26, 'erf_inv': 27, 'cbrt': 28, 'pow': 29, 'lgamma': 30, 'digamma': 31,
}
GEMM_MODE = {'f32': 0, 'bf16x3': 1}
BINOP = {'mul': 0, 'div': 1, 'add': 2, 'sub': 3, 'min': 4, 'max': 5}

_lib = None


class FolxHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load the kernel library once; raise loudly if it is not there."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIBPATH):
        raise FolxHipError(
            f'{LIBPATH} not found: build the HIP kernels with `python -m folx_amd.build` '
            '(there is no CPU fallback)'
        )
    lib = ctypes.CDLL(LIBPATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    mode = os.environ.get('FOLX_AMD_GEMM')
    if mode is not None:
        if mode not in GEMM_MODE:
            raise FolxHipError(f'FOLX_AMD_GEMM={mode!r}: expected one of {sorted(GEMM_MODE)}')
        lib.folx_hip_set_gemm_mode(GEMM_MODE[mode])
    _lib = lib
    return lib


def check(code: int, what: str):
    if code != OK:
        msg = load().folx_hip_strerror(code).decode()
        raise FolxHipError(f'{what}: {msg} (code {code})')

"""The C-ABI library loads and exports every symbol include/folx_hip.h declares; argument
checks reject bad calls before anything is launched (no GPU needed: nothing computes)."""

import ctypes
import os

import pytest

import __graft_entry__ as entry
from folx_amd import _lib


@pytest.fixture(scope='module')
def lib():
    if not os.path.exists(_lib.LIBPATH):
        from folx_amd import build

        build.build(verbose=False)
    return _lib.load()


def test_exports_every_declared_symbol(lib):
    declared = entry.declared_symbols()
    assert len(declared) >= 12
    assert set(declared) == set(_lib.SIGNATURES)
    for name in declared:
        assert getattr(lib, name) is not None


def test_gemm_mode_switch(lib):
    """The mode is a host-side flag: setting and reading it needs no GPU."""
    if 'FOLX_AMD_GEMM' not in os.environ:
        assert lib.folx_hip_get_gemm_mode() == _lib.GEMM_MODE['f32']  # the default
    before = lib.folx_hip_get_gemm_mode()
    assert lib.folx_hip_set_gemm_mode(_lib.GEMM_MODE['bf16x3']) == _lib.OK
    assert lib.folx_hip_get_gemm_mode() == _lib.GEMM_MODE['bf16x3']
    assert lib.folx_hip_set_gemm_mode(7) == _lib.EINVAL
    assert lib.folx_hip_get_gemm_mode() == _lib.GEMM_MODE['bf16x3']  # unchanged by the refused call
    assert lib.folx_hip_set_gemm_mode(_lib.GEMM_MODE['f32']) == _lib.OK
    assert lib.folx_hip_get_gemm_mode() == _lib.GEMM_MODE['f32']
    assert lib.folx_hip_set_gemm_mode(before) == _lib.OK


def test_version_and_strerror(lib):
    assert lib.folx_hip_version() >= 100
    assert lib.folx_hip_strerror(0) == b'ok'
    for code in (-1, -2, -3, -99):
        assert len(lib.folx_hip_strerror(code)) > 0


def test_argument_checks_return_error_codes(lib):
    null = ctypes.c_void_p(None)
    # negative sizes / null pointers -> EINVAL, nothing launched
    assert lib.folx_hip_dense_fwdlap(*([null] * 12), 4, 1, 8, 8) == _lib.EINVAL
    assert lib.folx_hip_dense_fwdlap(*([null] * 12), -1, 1, 8, 8) == _lib.EINVAL
    assert lib.folx_hip_elementwise_fwdlap(null, 99, 0.0, null, null, null, null, null, null, 4, 1) == _lib.EINVAL
    assert lib.folx_hip_elementwise_fwdlap(null, 0, 0.0, null, null, null, null, null, null, 4, 1) == _lib.EINVAL
    assert lib.folx_hip_binary_fwdlap(null, 0, null, null, null, null, null, null, null, null, null, null, 1, 1, 1) == _lib.EINVAL
    assert lib.folx_hip_rows_affine(null, null, null, 1, 1, null, null, 1.0, 1.0, null) == _lib.EINVAL
    assert lib.folx_hip_reduce_sum(null, null, null, 1, 1, -1, 1, 1.0) == _lib.EINVAL
    assert lib.folx_hip_slogdet_fwdlap(null, null, null, null, null, null, null, null, 4, 0, 1) == _lib.EINVAL
    assert lib.folx_hip_layernorm_fwdlap(*([null] * 9), 4, 8, 1, 1e-5) == _lib.EINVAL
    assert lib.folx_hip_mhsa_fwdlap(*([null] * 15), 1, 8, 1, 8, 1) == _lib.EINVAL
    assert lib.folx_hip_mhsea_fwdlap(*([null] * 18), 1, 8, 1, 8, 1) == _lib.EINVAL
    assert lib.folx_hip_dense_act_fwdlap(null, 0, 0.0, *([null] * 11), 4, 1, 8, 8, null, 0) == _lib.EINVAL
    assert lib.folx_hip_dense_act_workspace_bytes(-1, 1, 8, 8) == _lib.EINVAL
    assert lib.folx_hip_mhsa_sparse_fwdlap(*([null] * 14), 1, 8, 1, 8, 3) == _lib.EINVAL
    assert lib.folx_hip_mul_sparse_fwdlap(*([null] * 11), 8, 4, 2, 1) == _lib.EINVAL
    assert lib.folx_hip_mul_sparse_fwdlap(*([null] * 11), 9, 4, 2, 1) == _lib.EINVAL       # S not a multiple of S_w
    assert lib.folx_hip_exp_envelope_fwdlap(*([null] * 9), 4, 2, 8, 1) == _lib.EINVAL
    assert lib.folx_hip_slogdet_scaled_fwdlap(*([null] * 12), 1, 1, 4, 1, 16, 0, 4, 16, 16, 1) == _lib.EINVAL
    assert lib.folx_hip_dense_rows_fwdlap(*([null] * 12), 4, 1, 8, 8, 1, 1) == _lib.EINVAL
    assert lib.folx_hip_dot_two_fwdlap(*([null] * 10), 1, 1, 4, 4, 4, 1, null) == _lib.EINVAL
    assert lib.folx_hip_reduce_max(null, null, null, 2, 3, 4) == _lib.EINVAL
    assert lib.folx_hip_reduce_max(null, null, null, -2, 3, 4) == _lib.EINVAL
    assert lib.folx_hip_gather_reduce_rows(null, null, null, null, 2, 2, 1, 1, 4, 4, 1, 1, 1.0) == _lib.EINVAL
    assert lib.folx_hip_gather_cols(null, null, null, null, 2, 4, 4, 1, 1) == _lib.EINVAL
    assert lib.folx_hip_gather_cols(null, null, null, null, -2, 4, 4, 1, 1) == _lib.EINVAL
    assert lib.folx_hip_scatter_add_rows(null, null, null, null, 2, 4, 1, 4, 1) == _lib.EINVAL
    assert lib.folx_hip_slogdet_strided_fwdlap(*([null] * 8), 1, 1, 4, 1, 16, 16, 4, 16) == _lib.EINVAL
    assert lib.folx_hip_sparse_slogdet_fwdlap(*([null] * 11), 1, 4, 1, 1, 1, 1, 0) == _lib.EINVAL
    assert lib.folx_hip_inv_values(null, null, null, null, null, 1, 4) == _lib.EINVAL
    assert lib.folx_hip_trace_pair(null, null, null, null, 1, 4) == _lib.EINVAL
    assert lib.folx_hip_trace_pair(null, null, null, null, -1, 4) == _lib.EINVAL
    assert lib.folx_hip_inv_fwdlap(*([null] * 7), 1, 4, 1) == _lib.EINVAL
    assert lib.folx_hip_inv_fwdlap(*([null] * 7), -1, 4, 1) == _lib.EINVAL
    assert lib.folx_hip_solve_fwdlap(*([null] * 10), 1, 4, 1, 1) == _lib.EINVAL
    assert lib.folx_hip_solve_fwdlap(*([null] * 10), 1, 0, 1, 1) == _lib.EINVAL
    # empty problems are fine and launch nothing
    assert lib.folx_hip_dense_fwdlap(*([null] * 12), 0, 1, 8, 8) == _lib.OK
    assert lib.folx_hip_elementwise_fwdlap(null, 0, 0.0, null, null, null, null, null, null, 0, 1) == _lib.OK
    assert lib.folx_hip_gather_rows(null, null, null, null, 1, 0, 1, 4, 4, 4) == _lib.OK


def test_unsupported_sizes(lib):
    one = ctypes.c_void_p(16)  # non-null, never dereferenced: the size check comes first
    assert lib.folx_hip_slogdet_fwdlap(None, one, one, one, one, one, one, one, 4, 33, 1) == _lib.ENOTSUP
    assert lib.folx_hip_mhsa_fwdlap(None, *([one] * 9), None, None, one, one, one, 1, 65, 1, 8, 1) == _lib.ENOTSUP
    assert lib.folx_hip_mhsa_fwdlap(None, *([one] * 9), None, None, one, one, one, 1, 8, 1, 6, 1) == _lib.ENOTSUP
    assert lib.folx_hip_layernorm_fwdlap(None, one, one, one, None, None, one, one, one, 4, 6, 1, 1e-5) == _lib.ENOTSUP
    assert lib.folx_hip_layernorm_fwdlap(None, one, one, one, None, None, one, one, one, 4, 2048, 1, 1e-5) == _lib.ENOTSUP
    # fused / structure-aware entry points outside the sizes they are built for: the caller takes
    # the general rules instead
    assert lib.folx_hip_dense_act_fwdlap(None, 0, 0.0, *([one] * 5), None, None, None, *([one] * 3), 4, 1, 6, 8, None, 0) == _lib.ENOTSUP     # K % 4
    assert lib.folx_hip_dense_act_fwdlap(None, 0, 0.0, *([one] * 5), None, None, None, *([one] * 3), 4, 1, 256, 8, None, 0) == _lib.ENOTSUP   # K > 128
    assert lib.folx_hip_dense_act_fwdlap(None, 3, 0.0, *([one] * 5), None, None, None, *([one] * 3), 4, 1, 8, 8, None, 0) == _lib.ENOTSUP     # log: not fused
    assert lib.folx_hip_dense_act_workspace_bytes(64, 4, 8, 200) == _lib.ENOTSUP
    assert lib.folx_hip_dense_act_workspace_bytes(1 << 20, 4, 100, 100) == 0                                  # no split
    assert lib.folx_hip_dense_act_workspace_bytes(64, 64, 256, 256) == 2 * 64 * 256 * 4     # wide: 2 groups of 32 rows
    assert lib.folx_hip_dense_act_workspace_bytes(64, 33, 256, 256) == 3 * 64 * 256 * 4     # wide: 3 groups of 16 rows
    assert lib.folx_hip_dense_act_workspace_bytes(60, 33, 256, 256) == 2 * 60 * 256 * 4     # rows % 8: groups of 32
    assert lib.folx_hip_dense_act_workspace_bytes(63, 33, 256, 256) == _lib.ENOTSUP         # wide: rows % 4
    assert lib.folx_hip_dense_act_workspace_bytes(64, 33, 200, 256) == _lib.ENOTSUP         # wide: K % 16
    assert lib.folx_hip_dense_act_fwdlap(None, 0, 0.0, *([one] * 5), None, None, None, *([one] * 3), 64, 33, 256, 256, None, 0) == _lib.EINVAL  # no workspace
    assert lib.folx_hip_dense_act_fwdlap(None, 0, 0.0, *([one] * 11), 64, 33, 256, 256, one, 1 << 30) == _lib.ENOTSUP  # skip connection on a wide layer
    assert lib.folx_hip_dense_act_fwdlap(None, 0, 0.0, *([one] * 5), one, None, None, *([one] * 3), 4, 1, 8, 8, None, 0) == _lib.EINVAL    # part of a residual
    assert lib.folx_hip_reduce_sum_window(None, one, one, 2, 3, 8, 5, 9, 4, 1.0) == _lib.EINVAL   # window past the axis
    assert lib.folx_hip_reduce_sum_window(None, one, one, 2, 3, 8, 5, 4, 4, 1.0) == _lib.EINVAL   # hi < lo
    # Jacobian operand in parts: host arrays of pointers, widths and broadcast flags
    ptrs, wd, bc = (ctypes.c_void_p * 2)(16, 32), (ctypes.c_int32 * 2)(16, 32), (ctypes.c_int32 * 2)(0, 1)
    parts = lambda wd_, R, group, ws, nb: lib.folx_hip_dense_act_parts_fwdlap(
        None, 0, 0.0, one, one, 2, ptrs, wd_, bc, group, one, one, None, None, None, None, None, None, one, one, one, R, 33,
        256, ws, nb)
    assert parts(wd, 64, 4, None, 0) == _lib.EINVAL                                  # no workspace
    assert parts((ctypes.c_int32 * 2)(16, 24), 64, 4, one, 1 << 30) == _lib.ENOTSUP  # width % 16
    assert parts(wd, 64, 5, one, 1 << 30) == _lib.ENOTSUP                            # rows % group
    assert parts(wd, 64, 0, one, 1 << 30) == _lib.EINVAL
    assert lib.folx_hip_dense_act_parts_fwdlap(None, 0, 0.0, one, one, 2, ptrs, wd, bc, 4, one, one, one, None, None,
                                               None, None, None, one, one, one, 64, 33, 256, one, 1 << 30) == _lib.EINVAL  # part of a residual
    assert lib.folx_hip_dense_act_parts_fwdlap(None, 0, 0.0, one, one, 2, ptrs, wd, bc, 4, one, one, None, None, None,
                                               one, one, None, one, one, one, 64, 33, 256, one, 1 << 30) == _lib.EINVAL  # part of a pre-activation term
    # LayerNorm + dense (+ activation): act = -1 means none
    assert lib.folx_hip_norm_dense_workspace_bytes(64, 33, 256, 256, -1) > 2 * 64 * 256 * 4
    assert lib.folx_hip_norm_dense_workspace_bytes(64, 33, 256, 256, 0) > lib.folx_hip_norm_dense_workspace_bytes(64, 33, 256, 256, -1)
    assert lib.folx_hip_norm_dense_workspace_bytes(64, 33, 1024, 256, -1) == _lib.ENOTSUP    # K > 512
    assert lib.folx_hip_norm_dense_workspace_bytes(64, 33, 256, 128, -1) == _lib.ENOTSUP     # narrow layer
    assert lib.folx_hip_norm_dense_workspace_bytes(64, 33, 256, 256, 3) == _lib.ENOTSUP      # log: not fused
    assert lib.folx_hip_norm_dense_workspace_bytes(-1, 33, 256, 256, -1) == _lib.EINVAL
    nd = lambda act, R, K, N, ws, nb: lib.folx_hip_norm_dense_fwdlap(None, act, 0.0, one, one, one, one, one, 1e-5, one,
                                                                    one, one, one, one, R, 33, K, N, ws, nb)
    assert nd(-1, 64, 256, 256, None, 0) == _lib.EINVAL        # no workspace
    assert nd(-1, 62, 256, 256, one, 1 << 30) == _lib.ENOTSUP  # rows % 4
    assert nd(3, 64, 256, 256, one, 1 << 30) == _lib.ENOTSUP   # log: not fused
    # the same rule on the library's own scratch array: size checks come before any GPU call
    nds = lambda act, R, K, N: lib.folx_hip_norm_dense_static_fwdlap(None, act, 0.0, one, one, one, one, one, 1e-5, one,
                                                                     one, one, one, one, R, 33, K, N)
    assert nds(-1, 62, 256, 256) == _lib.ENOTSUP      # rows % 4
    assert nds(3, 64, 256, 256) == _lib.ENOTSUP       # log: not fused
    assert nds(-1, -4, 256, 256) == _lib.EINVAL
    assert lib.folx_hip_norm_dense_workspace_bytes(1 << 17, 33, 256, 256, 0) > _lib.STATIC_SCRATCH_BYTES
    assert nds(0, 1 << 17, 256, 256) == _lib.ESCRATCH  # beyond the 64 MiB array: refused, nothing launched
    assert b'scratch' in lib.folx_hip_strerror(_lib.ESCRATCH)
    assert lib.folx_hip_dense_act_workspace_bytes(2000, 400, 100, 100) > 0                                    # rows split
    assert lib.folx_hip_mhsa_sparse_fwdlap(None, *([one] * 13), 1, 65, 1, 8, 3) == _lib.ENOTSUP
    assert lib.folx_hip_mhsa_sparse_fwdlap(None, *([one] * 13), 1, 8, 1, 6, 3) == _lib.ENOTSUP
    assert lib.folx_hip_mul_sparse_fwdlap(None, *([one] * 10), 8, 4, 2, 9) == _lib.ENOTSUP
    assert lib.folx_hip_exp_envelope_fwdlap(None, *([one] * 8), 4, 9, 8, 1) == _lib.ENOTSUP
    assert lib.folx_hip_exp_envelope_fwdlap(None, *([one] * 8), 4, 2, 6, 1) == _lib.ENOTSUP
    assert lib.folx_hip_slogdet_scaled_fwdlap(None, *([one] * 11), 1, 1, 32, 1, 1024, 0, 32, 1024, 1024, 1) == _lib.ENOTSUP
    assert lib.folx_hip_slogdet_scaled_fwdlap(None, *([one] * 11), 1, 1, 8, 1, 64, 0, 8, 64, 64, 5) == _lib.ENOTSUP


def test_product_fails_loudly_without_gpu():
    import numpy as np
    import torch

    import folx_amd
    from folx_amd import numpy as fnp

    if torch.cuda.is_available():
        pytest.skip('GPU present')
    with pytest.raises(_lib.FolxHipError):
        folx_amd.forward_laplacian(lambda x: fnp.tanh(x), 0)(np.zeros(3, np.float32))

"""The entry point that allocates nothing: ``folx_hip_norm_dense_static_fwdlap`` (LayerNorm +
dense (+ activation) on the library's own scratch array) against ``folx_hip_norm_dense_fwdlap``
with a caller-owned workspace, both called through the C ABI.  The two run the same kernels, so
the outputs must agree bit for bit; the oracle chain is checked on the second, smaller call.
"""

import ctypes

import numpy as np
import pytest
import torch

from tolerances import assert_triplet

pytestmark = pytest.mark.gpu


def _ptr(t):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _inputs(seed, R, P, Kd, N):
    g = torch.Generator(device='cuda').manual_seed(seed)
    rn = lambda *s: torch.randn(*s, device='cuda', generator=g)
    x, J, L = rn(R, Kd) + 0.5, rn(P, R, Kd), rn(R, Kd)
    gam, bet = 1 + 0.2 * rn(Kd), 0.2 * rn(Kd)
    W, b = rn(Kd, N) / np.sqrt(Kd), rn(N)
    return x, J, L, gam, bet, W, b


def _call(lib, static, act, x, J, L, gam, bet, W, b, R, P, Kd, N):
    from folx_amd import _lib

    y, yj, yl = (torch.full((R, N), float('nan'), device='cuda'), torch.full((P, R, N), float('nan'), device='cuda'),
                 torch.full((R, N), float('nan'), device='cuda'))
    st = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    head = (st, act, 0.0, _ptr(x), _ptr(J), _ptr(L), _ptr(gam), _ptr(bet), 1e-5, _ptr(W), _ptr(b), _ptr(y), _ptr(yj),
            _ptr(yl), R, P, Kd, N)
    if static:
        rc = lib.folx_hip_norm_dense_static_fwdlap(*head)
    else:
        nb = int(lib.folx_hip_norm_dense_workspace_bytes(R, P, Kd, N, act))
        assert nb > 0
        ws = torch.empty(nb // 4, device='cuda')
        rc = lib.folx_hip_norm_dense_fwdlap(*head, _ptr(ws), nb)
    _lib.check(rc, 'norm_dense' + ('_static' if static else ''))
    torch.cuda.synchronize()
    return y, yj, yl


def test_static_scratch_entry_point_matches_workspace_entry_point():
    from oracle import backend as ob
    from oracle import rules

    from folx_amd import _lib

    lib = _lib.load()
    torch.cuda.set_device(0)
    # two calls in a row on the shared scratch array, the second one smaller: what the first
    # call left behind must not reach the second call's results
    for seed, (R, P, Kd, N, act) in enumerate([(2048, 96, 256, 256, _lib.ACT['tanh']), (96, 40, 64, 192, -1)]):
        print(f'case norm_dense_static R={R} P={P} K={Kd} N={N} act={act}', flush=True)
        assert int(lib.folx_hip_norm_dense_workspace_bytes(R, P, Kd, N, act)) <= _lib.STATIC_SCRATCH_BYTES
        ins = _inputs(11 + seed, R, P, Kd, N)
        want = _call(lib, False, act, *ins, R, P, Kd, N)
        x, J, L, gam, bet, W, b = ins
        y, yj, yl = torch.empty(R, N, device='cuda'), torch.empty(P, R, N, device='cuda'), torch.empty(R, N, device='cuda')
        held = torch.cuda.memory_allocated()
        rc = lib.folx_hip_norm_dense_static_fwdlap(
            ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), act, 0.0, _ptr(x), _ptr(J), _ptr(L), _ptr(gam),
            _ptr(bet), 1e-5, _ptr(W), _ptr(b), _ptr(y), _ptr(yj), _ptr(yl), R, P, Kd, N)
        _lib.check(rc, 'norm_dense_static')
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == held  # nothing was taken from torch's allocator during the call
        for got, ref, nm in zip((y, yj, yl), want, ('x', 'jac', 'lap')):
            assert torch.equal(got, ref), f'{nm}: static-scratch result differs from the workspace entry point'
    # the smaller case against the oracle's chain of rules (fp64)
    f64 = lambda t: t.cpu().numpy().astype(np.float64)
    h = ob.layer_norm(ob.OArr(f64(x), f64(J), f64(L)), f64(gam), f64(bet), 1e-5)
    ref = rules.dense_rule(h.x, h.J, h.lap, f64(W), f64(b))
    assert_triplet((y, yj, yl), ref, 'norm_dense_static vs oracle')


def test_static_scratch_rejects_what_does_not_fit():
    from folx_amd import _lib

    lib = _lib.load()
    one = ctypes.c_void_p(256)
    R, P, Kd, N = 32768, 96, 256, 256
    assert int(lib.folx_hip_norm_dense_workspace_bytes(R, P, Kd, N, 0)) > _lib.STATIC_SCRATCH_BYTES
    rc = lib.folx_hip_norm_dense_static_fwdlap(None, 0, 0.0, one, one, one, one, one, 1e-5, one, one, one, one, one, R, P,
                                               Kd, N)
    assert rc == _lib.ESCRATCH
    assert b'scratch' in lib.folx_hip_strerror(rc)

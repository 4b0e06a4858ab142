"""The traced front door (``folx_amd.forward_laplacian_torch``, the counterpart of the reference's jaxpr interpreter,
folx/interpreter.py:127-264): models written with plain torch against the Hessian trace of the same function by
torch AD in float64 -- on the CPU stand-ins at several thresholds, and on the GPU."""

import numpy as np
import pytest
import torch

import cpu_kernels
from bruteforce import brute_force
from tolerances import assert_lap, assert_val
from torch_models import MODELS

import folx_amd


def _leaves(out):
    return list(out) if isinstance(out, (tuple, list)) else [out]


def _check(name, thr, device):
    make, x = MODELS[name]()
    fl = folx_amd.forward_laplacian_torch(make(torch.float32), thr)
    xin = torch.as_tensor(x).to(device)
    outs = _leaves(folx_amd.vmap(fl)(xin))
    again = _leaves(folx_amd.vmap(fl)(xin))          # the second call reuses the traced graph
    assert len(fl.graphs) == 1
    f64 = make(torch.float64)
    for i, (out, out2) in enumerate(zip(outs, again)):
        pick = (lambda t, i=i: _leaves(f64(t))[i])
        by, bJ, bL = brute_force(pick, x.astype(np.float64))
        J = out.jacobian.dense_array
        if J.shape[0] < bJ.shape[0]:
            assert not np.abs(bJ[J.shape[0]:]).any()
            bJ = bJ[: J.shape[0]]
        assert_val(out.x, by, f'{name} output {i} value')
        assert_val(J, bJ.reshape(tuple(J.shape)), f'{name} output {i} jacobian')
        assert_lap(out.laplacian, bL, f'{name} output {i} laplacian')
        assert torch.equal(out.x, out2.x) and torch.equal(out.laplacian, out2.laplacian)


@pytest.mark.parametrize('name', sorted(MODELS))
@pytest.mark.parametrize('thr', [0, 3, 100])
def test_torch_models_on_the_host_logic(name, thr, monkeypatch):
    cpu_kernels.install(monkeypatch)
    from folx_amd import sparse_ops

    sparse_ops.clear_caches()
    _check(name, thr, 'cpu')


def test_unknown_operation_gets_the_generic_rule(monkeypatch, caplog):
    """An ATen operation outside the table is wrapped on the fly, with a warning (folx/wrapped_functions.py:609-614)."""
    cpu_kernels.install(monkeypatch)
    x = np.random.default_rng(3).normal(size=(2, 5)).astype(np.float32)
    f = lambda t: torch.special.sinc(t).sum() + torch.tanh(t).sum()
    with caplog.at_level('WARNING'):
        out = folx_amd.vmap(folx_amd.forward_laplacian_torch(f, 0))(x)
    assert any('no forward-Laplacian rule' in r.message for r in caplog.records)
    by, bJ, bL = brute_force(f, x.astype(np.float64))
    np.testing.assert_allclose(out.x.numpy(), by, rtol=1e-5)
    np.testing.assert_allclose(out.laplacian.numpy(), bL, rtol=1e-4, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(MODELS))
@pytest.mark.parametrize('thr', [0, 3])
def test_torch_models_on_the_gpu(name, thr):
    print(f'traced torch model {name} thr={thr}', flush=True)
    _check(name, thr, 'cuda')

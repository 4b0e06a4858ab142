"""HIP-graph replay of a forward-Laplacian evaluation: every replay must equal the eager
result, with eager work and synchronisations between the replays."""

import numpy as np
import pytest
import torch

import folx_amd
from folx_amd import workloads as wl

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('name', ['ferminet', 'psiformer'])
def test_graph_replay_equals_eager(name):
    if name == 'ferminet':
        cfg = wl.FermiNetConfig(n_elec=6, n_nuc=2, n_layers=3, w1=16, w2=8, n_det=3)
        p = wl.to_device(wl.ferminet_params(cfg), torch.device('cuda'))
        f = lambda r: wl.ferminet_forward(p, r)
    else:
        cfg = wl.PsiFormerConfig(n_elec=6, n_nuc=2, n_layers=2, n_heads=2, head_dim=8, width=16, mlp_width=16, n_det=3)
        p = wl.to_device(wl.psiformer_params(cfg), torch.device('cuda'))
        f = lambda r: wl.psiformer_forward(p, r)
    eager = folx_amd.vmap(folx_amd.forward_laplacian(f, 6))
    fast = folx_amd.jit(eager)
    for rep in range(6):  # call 1 eager, call 2 captures, calls 3+ replay
        print(f'case graph {name} rep {rep}', flush=True)
        x = torch.as_tensor(wl.sample_electrons(32, cfg.n_elec, 1.0, seed=10 + rep)).cuda()
        ref = eager(x)
        torch.cuda.synchronize()
        out = fast(x)
        torch.cuda.synchronize()
        assert torch.equal(out.x, ref.x)
        assert torch.equal(out.jacobian.dense_array, ref.jacobian.dense_array)
        assert torch.equal(out.laplacian, ref.laplacian)
        # unrelated eager work between replays
        junk = eager(torch.as_tensor(wl.sample_electrons(8, cfg.n_elec, 1.0, seed=99)).cuda())
        assert torch.isfinite(junk.x).all()


def test_jit_weights_in_place_and_invalidate():
    """The graph reads device weights by address: an in-place update is seen by the next replay;
    a weight rebound to another tensor needs ``invalidate()``, after which the function is captured
    again."""
    from folx_amd import numpy as fnp

    g = torch.Generator(device='cuda').manual_seed(2)
    box = {'W': torch.randn(6, 8, device='cuda', generator=g) / 2}
    fn = lambda r: fnp.sum(fnp.tanh(fnp.dot(r, box['W'])))
    eager = folx_amd.vmap(folx_amd.forward_laplacian(fn, 0))
    jitted = folx_amd.jit(eager)
    x = torch.randn(5, 3, 6, device='cuda', generator=g)
    for _ in range(3):
        out = jitted(x)
    assert torch.equal(out.laplacian, eager(x).laplacian)
    box['W'].mul_(1.5)                      # in place: same address
    assert torch.equal(jitted(x).laplacian, eager(x).laplacian)
    box['W'] = box['W'] * 0.5               # rebound: another tensor
    stale = jitted(x)
    assert not torch.equal(stale.laplacian, eager(x).laplacian)
    jitted.invalidate()
    for _ in range(3):
        out = jitted(x)
    assert torch.equal(out.laplacian, eager(x).laplacian)
    assert torch.equal(out.jacobian.dense_array, eager(x).jacobian.dense_array)

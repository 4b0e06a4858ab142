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


def test_jit_in_place_weight_update_reaches_every_part_of_a_concatenated_layer():
    """A layer that reads a concatenation part by part contracts its per-position parts with a copy of
    their rows of ``W`` (two kept row ranges here) and its per-walker part with a view of its rows.  With
    ``W`` a device tensor the caller updates in place, a replay must read the new rows in every part: the
    copy is made on every call (and so recorded in the graph), never served from a cache."""
    from folx_amd import numpy as fnp

    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(4)
    n = 16                                                           # 48 Jacobian rows: full groups of 16
    W0 = torch.randn(3, 16, device='cuda', generator=g)
    Wm = torch.randn(16, 32, device='cuda', generator=g) / 4
    box = {'W': torch.randn(16 + 16 + 32, 136, device='cuda', generator=g) / 6}

    def fn(r):
        e = fnp.dot(r, W0)                                           # (n, 16)
        m = fnp.mean(fnp.tanh(e), axis=0)                            # (16,) per walker
        h = fnp.tanh(fnp.dot(fnp.add(e, m), Wm))                     # (n, 32)
        f = fnp.concatenate([e, fnp.broadcast_to(m, (n, 16)), h], axis=-1)
        return fnp.sum(fnp.tanh(fnp.dot(f, box['W'])))

    eager = folx_amd.vmap(folx_amd.forward_laplacian(fn, 0))
    jitted = folx_amd.jit(eager)
    x = torch.randn(5, n, 3, device='cuda', generator=g)
    print('case jit concat layer, in-place weight update', flush=True)
    with K.LaunchTimer() as lt:
        eager(x)
    # the fused layer contracts the 16 + 32 per-position features only: its copy of two row ranges of W is in use
    assert any(entry == 'dense_act_fwdlap' and key[3] == 48 for (entry, key) in lt.summary()), lt.summary()
    for _ in range(3):
        out = jitted(x)
    assert torch.equal(out.laplacian, eager(x).laplacian)
    before = out.laplacian.clone()
    box['W'].mul_(1.5)                                               # same address, new values
    for _ in range(2):
        out = jitted(x)
        ref = eager(x)
        assert torch.equal(out.laplacian, ref.laplacian)
        assert torch.equal(out.jacobian.dense_array, ref.jacobian.dense_array)
    assert not torch.equal(out.laplacian, before)

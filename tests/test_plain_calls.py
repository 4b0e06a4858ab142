"""Fusion without annotations, host side (CPU stand-ins for the kernels): the benchmark models
written with plain calls (``folx_amd/workloads.py``) issue exactly the kernel calls of the forms
that spell every fusion out (``tests/annotated_workloads.py``) and return the same numbers; and a
deferred value that nobody absorbs is evaluated by the ordinary rule."""

import numpy as np
import pytest
import torch

import annotated_workloads as ann
import cpu_kernels
from oracle import backend as ob

import folx_amd
from folx_amd import numpy as fnp
from folx_amd import workloads as wl


@pytest.fixture(autouse=True)
def _cpu(monkeypatch):
    cpu_kernels.install(monkeypatch)
    from folx_amd import sparse_ops

    sparse_ops.clear_caches()


def traced(fn, x, thr):
    """(result, [(kernel, shapes of its tensor arguments), ...])"""
    import folx_amd.kernels as K

    calls, orig = [], {}

    def shapes(v):
        if isinstance(v, torch.Tensor):
            return tuple(v.shape)
        if isinstance(v, (tuple, list)):
            return tuple(shapes(t) for t in v)
        return v if isinstance(v, (int, float, str, bool, type(None))) else type(v).__name__

    for name in cpu_kernels.KERNEL_NAMES:
        orig[name] = getattr(K, name)
        setattr(K, name, (lambda nm, f: lambda *a, **k: (calls.append((nm, shapes(a), shapes(tuple(k.values())))), f(*a, **k))[1])(name, orig[name]))
    try:
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
    finally:
        for name, f in orig.items():
            setattr(K, name, f)
    return out, calls


FORMS = {
    'mlp': (wl.mlp_forward, ann.mlp_forward),
    'psiformer': (wl.psiformer_forward, ann.psiformer_forward),
    'ferminet': (wl.ferminet_forward, ann.ferminet_forward),
}


@pytest.mark.parametrize('name,thr', [('mlp_dense', 0), ('mlp_sparse', 4), ('ferminet16', 6), ('ferminet16', 0),
                                      ('psiformer32', 6), ('psiformer32', 0)])
def test_plain_calls_issue_the_kernel_calls_of_the_annotated_form(name, thr):
    """Full model widths, one walker: the same kernel calls with the same shapes,
    same results -- and the fused rules are among them."""
    forward, p, cfg, _, sigma, _ = wl.build(name)
    plain_fn, ann_fn = FORMS['mlp' if name.startswith('mlp') else name.rstrip('0123456789')]
    assert forward is plain_fn
    x = wl.sample_inputs(name, 1, seed=3)
    got, calls = traced(lambda xp, t: plain_fn(p, t, xp), x, thr)
    want, calls_ann = traced(lambda xp, t: ann_fn(p, t, xp), x, thr)
    # deferred evaluation may run independent rules in another order; the set of calls is the same
    key = lambda c: repr(c)
    assert sorted(c[0] for c in calls) == sorted(c[0] for c in calls_ann)
    assert sorted(calls, key=key) == sorted(calls_ann, key=key)
    assert torch.equal(got.x, want.x) and torch.equal(got.laplacian, want.laplacian)
    assert torch.equal(got.jacobian.dense_array, want.jacobian.dense_array)
    used = [c[0] for c in calls]
    if name.startswith('psiformer'):
        assert used.count('norm_dense') == (3 * 3 + 4 if thr else 4 * 4), used      # LayerNorm inside q, k, v and the MLP
        assert used.count('layernorm') == (1 if thr else 0), used                  # only the sparse first layer's
        assert not any(c[0] == 'elementwise' and c[1][0] == 'tanh' for c in calls)  # tanh always in a product's epilogue
        if thr:  # matrix rows read in place (row axis 1 of (walker, electron, det, orbital)), factor on load
            assert all(len(c[1]) == 5 and c[1][3] == 1 and c[1][4] is not None for c in calls if c[0] == 'slogdet')
    if name == 'ferminet16' and thr:
        assert used.count('dense_act_parts') == 3 and used.count('dense_act') >= 3, used
        assert any(c[0] == 'reduce_sum' and c[1][-1] == (0, 8) for c in calls)   # spin means read their window in place
    if name.startswith('mlp'):
        assert used.count('dense_act') == 10 and 'elementwise' not in used, used


def test_deferred_values_nobody_absorbs():
    """Every deferred kind evaluated by the ordinary rule: results equal the float64 oracle."""
    x = np.random.default_rng(4).normal(size=(2, 6, 16)).astype(np.float32)
    W = (np.random.default_rng(5).normal(size=(16, 16)) / 4).astype(np.float32)
    g, b = np.linspace(0.5, 1.5, 16).astype(np.float32), np.linspace(-1, 1, 16).astype(np.float32)

    def fn(xp, t):
        ln = xp.layer_norm(t, g, b, 1e-5)                     # consumed by exp, not by a product
        d = xp.dot(t, W)                                      # consumed by a slice and a reshape
        sl = xp.getitem(d, (slice(1, 4),))                    # consumed by exp (not a product or sum)
        mu = xp.multiply(xp.exp(ln), ln)                      # consumed by sum, not by slogdet
        tr = xp.transpose(xp.reshape(d, (6, 4, 4)), (1, 0, 2))  # consumed by sum
        bc = xp.broadcast_to(xp.mean(t, axis=0), (6, 16))     # consumed by add
        cat = xp.concatenate([t, bc], axis=-1)                # consumed by tanh
        return xp.add(xp.add(xp.sum(xp.exp(sl)), xp.sum(mu)), xp.add(xp.sum(tr), xp.sum(xp.tanh(cat))))

    for thr in (0, 16):
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
        ref = fn(ob, ob.init_state(x, dtype=np.float64))
        np.testing.assert_allclose(out.x.numpy(), ref.x, rtol=1e-5)
        np.testing.assert_allclose(out.jacobian.dense_array.numpy(), ref.J, rtol=1e-4, atol=1e-5)
        np.testing.assert_allclose(out.laplacian.numpy(), ref.lap, rtol=1e-4, atol=1e-4)


def test_deferred_value_behaves_like_a_triplet():
    x = np.random.default_rng(6).normal(size=(2, 5, 8)).astype(np.float32)
    W = np.eye(8, dtype=np.float32)
    seen = {}

    def fn(t):
        d = fnp.dot(t, W)
        seen['type'] = type(d).__name__
        seen['shape'], seen['ndim'] = d.shape, d.ndim
        e = d + 1.0                       # operator sugar on the handle
        seen['x'] = d.x.shape             # attribute access evaluates
        return (e * 2.0).sum()

    out = folx_amd.vmap(folx_amd.forward_laplacian(fn, 0))(x)
    assert seen == {'type': 'LazyDot', 'shape': (5, 8), 'ndim': 2, 'x': (2, 5, 8)}
    np.testing.assert_allclose(out.x.numpy(), 2.0 * (x.reshape(2, -1).sum(1) + 40.0), rtol=1e-5)

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


def _both_front_doors(forward, params, x, thr, device):
    from folx_amd import torch_namespace as txp

    by_calls = folx_amd.vmap(folx_amd.forward_laplacian(lambda r: forward(params, r), thr))(torch.as_tensor(x).to(device))
    traced = folx_amd.vmap(folx_amd.forward_laplacian_torch(lambda r: forward(params, r, xp=txp), thr))(torch.as_tensor(x).to(device))
    J1, J2 = by_calls.jacobian.dense_array.cpu().numpy(), traced.jacobian.dense_array.cpu().numpy()
    scale = lambda a: max(1.0, float(np.abs(a).max()))
    np.testing.assert_allclose(traced.x.cpu().numpy(), by_calls.x.cpu().numpy(), rtol=2e-4, atol=2e-5 * scale(J1))
    np.testing.assert_allclose(J2, J1, rtol=5e-4, atol=1e-4 * scale(J1))
    np.testing.assert_allclose(traced.laplacian.cpu().numpy(), by_calls.laplacian.cpu().numpy(), rtol=5e-4,
                               atol=2e-4 * scale(by_calls.laplacian.cpu().numpy()))


@pytest.mark.parametrize('thr', [0, 6])
def test_benchmark_models_through_the_traced_front_door(thr, monkeypatch):
    """The benchmark architectures (small widths) as plain torch code (``folx_amd.torch_namespace``), traced, against the
    same models written with ``folx_amd.numpy`` calls."""
    from folx_amd import workloads as wl

    cpu_kernels.install(monkeypatch)
    psi = wl.PsiFormerConfig(n_elec=4, n_nuc=2, n_layers=2, n_heads=2, head_dim=4, width=8, mlp_width=8, n_det=2, orb_shift=1.5)
    fermi = wl.FermiNetConfig(n_elec=4, n_nuc=2, n_layers=3, w1=8, w2=4, n_det=2, orb_shift=1.5)
    for cfg, forward, make in ((psi, wl.psiformer_forward, wl.psiformer_params), (fermi, wl.ferminet_forward, wl.ferminet_params)):
        x = wl.sample_electrons(3, cfg.n_elec, 1.0, seed=5)
        _both_front_doors(forward, make(cfg), x, thr, 'cpu')
    params = wl.mlp_params(seed=0, in_dim=4, width=8, n_hidden=3)
    _both_front_doors(wl.mlp_forward, params, np.random.default_rng(0).normal(size=(3, 6, 4)).astype(np.float32), thr, 'cpu')


@pytest.mark.gpu
@pytest.mark.parametrize('thr', [0, 6])
def test_benchmark_models_through_the_traced_front_door_on_the_gpu(thr):
    from folx_amd import workloads as wl

    print(f'benchmark architectures through both front doors, thr={thr}', flush=True)
    psi = wl.PsiFormerConfig(n_elec=6, n_nuc=2, n_layers=2, n_heads=2, head_dim=8, width=16, mlp_width=16, n_det=3, orb_shift=1.5)
    fermi = wl.FermiNetConfig(n_elec=6, n_nuc=2, n_layers=3, w1=16, w2=8, n_det=3, orb_shift=1.5)
    for cfg, forward, make in ((psi, wl.psiformer_forward, wl.psiformer_params), (fermi, wl.ferminet_forward, wl.ferminet_params)):
        x = wl.sample_electrons(5, cfg.n_elec, 1.0, seed=5)
        _both_front_doors(forward, make(cfg), x, thr, 'cuda')


@pytest.mark.gpu
def test_traced_model_under_graph_replay():
    """``folx_amd.jit`` around a traced model: replays return the bits of the eager evaluation."""
    make, x = MODELS['transformer_block']()
    fl = folx_amd.forward_laplacian_torch(make(torch.float32), 3)
    eager, fast = folx_amd.vmap(fl), folx_amd.jit(folx_amd.vmap(fl))
    for call in range(4):
        xin = torch.as_tensor(x + 0.01 * call).cuda()
        a, b = eager(xin), fast(xin)
        torch.cuda.synchronize()
        assert torch.equal(a.x, b.x) and torch.equal(a.laplacian, b.laplacian), f'call {call}'
        assert torch.equal(a.jacobian.dense_array, b.jacobian.dense_array), f'call {call}'


def _check_construct(name, thr, device, caplog):
    from torch_constructs import CONSTRUCTS, X

    fn, _ = CONSTRUCTS[name](torch.float32)
    _, fn_ad = CONSTRUCTS[name](torch.float64)
    with caplog.at_level('WARNING'):
        out = folx_amd.vmap(folx_amd.forward_laplacian_torch(fn, thr))(torch.as_tensor(X).to(device))
    assert not [r for r in caplog.records if 'no forward-Laplacian rule' in r.message], 'fell back to the generic rule'
    by, bJ, bL = brute_force(fn_ad, X.astype(np.float64))
    J = out.jacobian.dense_array
    if J.shape[0] < bJ.shape[0]:
        assert not np.abs(bJ[J.shape[0]:]).any()
        bJ = bJ[: J.shape[0]]
    assert_val(out.x, by, f'{name} value')
    assert_val(J, bJ.reshape(tuple(J.shape)), f'{name} jacobian')
    assert_lap(out.laplacian, bL, f'{name} laplacian')


def _construct_names():
    from torch_constructs import CONSTRUCTS

    return sorted(CONSTRUCTS)


@pytest.mark.parametrize('name', _construct_names())
@pytest.mark.parametrize('thr', [0, 6])
def test_everyday_torch_constructs_have_rules(name, thr, monkeypatch, caplog):
    """Functional calls, modules, linalg and indexing as they appear in ordinary torch code: every traced equation finds
    a rule of its own (no generic fallback), results against AD in float64."""
    cpu_kernels.install(monkeypatch)
    _check_construct(name, thr, 'cpu', caplog)


@pytest.mark.gpu
@pytest.mark.parametrize('name', _construct_names())
def test_everyday_torch_constructs_on_the_gpu(name, caplog):
    print(f'torch construct {name}', flush=True)
    _check_construct(name, 6, 'cuda', caplog)


def _named_function_model():
    from folx_amd import fx

    torch.manual_seed(3)
    W = torch.randn(4, 6) / 2
    layer = fx.named_function('test_gated_layer', lambda h, g: torch.tanh(h @ W.to(h)) * torch.sigmoid(g).sum())   # (the generic rule runs it where the data is)
    pair = fx.named_function('test_sin_cos_pair', lambda h: (torch.sin(h), torch.cos(h).sum(-1)))

    def model(x):
        s, c = pair(layer(x, x[:, 0]))
        return (s * c[:, None]).sum(0)

    return model, W


def _check_named_functions(device):
    """A function kept as one equation of the trace and looked up by NAME when the graph is evaluated
    (folx/interpreter.py:186-200): the generic rule without a registry entry, the registered rule with one."""
    from folx_amd import numpy as fnp

    model, W = _named_function_model()
    x = np.random.default_rng(0).normal(size=(2, 3, 4)).astype(np.float32)
    by, bJ, bL = brute_force(model, x.astype(np.float64))          # outside a trace the names are the plain functions
    fl = folx_amd.forward_laplacian_torch(model, 0)
    out = folx_amd.vmap(fl)(torch.as_tensor(x).to(device))
    (gm,) = fl.graphs.values()
    targets = [str(n.target) for n in gm.graph.nodes if n.op == 'call_function']
    assert 'folx_amd.test_gated_layer.default' in targets and 'folx_amd.test_sin_cos_pair.default' in targets
    assert not any('tanh' in t or 'sigmoid' in t for t in targets)          # the bodies are not in the trace
    assert_val(out.x, by, 'value')
    assert_val(out.jacobian.dense_array, bJ.reshape(tuple(out.jacobian.dense_array.shape)), 'jacobian')
    assert_lap(out.laplacian, bL, 'laplacian')
    seen = []

    def rule(args, kwargs, thr):            # a rule of the caller's own under the same name
        seen.append(len(args))
        h, g = args
        return fnp.multiply(fnp.tanh(fnp.dot(h, W.numpy())), fnp.sum(fnp.sigmoid(g)))

    folx_amd.register_function('test_gated_layer', rule)
    try:
        out2 = folx_amd.vmap(fl)(torch.as_tensor(x).to(device))
    finally:
        folx_amd.deregister_function('test_gated_layer')
    assert seen == [2]
    assert_val(out2.x, by, 'value by the registered rule')
    assert_lap(out2.laplacian, bL, 'laplacian by the registered rule')


def test_named_functions_are_single_equations_looked_up_by_name(monkeypatch):
    cpu_kernels.install(monkeypatch)
    _check_named_functions('cpu')


@pytest.mark.gpu
def test_named_functions_on_the_gpu():
    _check_named_functions('cuda')

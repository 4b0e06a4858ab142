"""The reference's per-rule tests (test/test_layers.py, real-valued halves) run as they are written there: one sample,
``forward_laplacian(f, sparsity)(x)`` at sparsity 0 and ``x.size``, value / Jacobian / Laplacian against AD in fp64
(test/laplacian_testcase.py:22-49, test/test_layers.py:653-666).  On the CPU the kernels are the test-only stand-ins
(host logic); the ``gpu`` half runs the same cases through the HIP library."""

import numpy as np
import pytest
import torch

import cpu_kernels
import reference_layer_cases as rc
from bruteforce import brute_force_single

import folx_amd
from folx_amd import numpy as fnp


def _check(name, thr_kind, device):
    f, g, x = rc.CASES[name]
    thr = 0 if thr_kind == 'dense' else x.size
    xin = torch.as_tensor(x).to(device) if device != 'cpu' else x
    y = folx_amd.forward_laplacian(f, thr)(xin)
    want_y, want_J, want_L = brute_force_single(g, x.astype(np.float64))
    # a triplet always carries a walker axis; the single-sample call gives it length one
    assert y.B == 1 and tuple(y.shape) == want_y.shape, (y.shape, want_y.shape)
    got_y = y.x[0].cpu().numpy().astype(np.float64)
    J = y.jacobian.dense_array[:, 0].cpu().numpy().astype(np.float64)
    # the dense Jacobian is truncated at the highest referenced input (test/test_layers.py:660-662)
    assert J.shape[0] <= want_J.shape[0]
    floor = lambda r: 2e-6 * max(1.0, float(np.abs(r).max()))    # noqa: E731   fp32 rounding at the result's scale
    np.testing.assert_allclose(got_y, want_y, rtol=2e-5, atol=floor(want_y), err_msg=name)        # rtol: laplacian_testcase.py:40
    np.testing.assert_allclose(J, want_J[:J.shape[0]], rtol=2e-5, atol=floor(want_J), err_msg=name)
    np.testing.assert_allclose(want_J[J.shape[0]:], 0.0, atol=0.0)
    np.testing.assert_allclose(y.laplacian[0].cpu().numpy().astype(np.float64), want_L, rtol=1e-4, atol=10 * floor(want_L),
                               err_msg=name)
    return y


@pytest.mark.parametrize('thr_kind', ['dense', 'sparse'])
@pytest.mark.parametrize('name', sorted(rc.CASES))
def test_reference_layer_case_host_logic(name, thr_kind, monkeypatch):
    cpu_kernels.install(monkeypatch)
    _check(name, thr_kind, 'cpu')


@pytest.mark.gpu
@pytest.mark.parametrize('thr_kind', ['dense', 'sparse'])
@pytest.mark.parametrize('name', sorted(rc.CASES))
def test_reference_layer_case_on_the_gpu(name, thr_kind):
    print(f'reference layer case {name} {thr_kind}', flush=True)
    _check(name, thr_kind, 'cuda')


def test_summation_has_no_laplacian_and_a_scalar_value(monkeypatch):
    """test/test_layers.py:25-36."""
    cpu_kernels.install(monkeypatch)
    for thr in (0, 10):
        y = folx_amd.forward_laplacian(fnp.sum, thr)(rc.X10)
        assert tuple(y.shape) == () and float(y.laplacian[0]) == 0.0
        np.testing.assert_allclose(y.jacobian.dense_array[:, 0].numpy(), np.ones(10, np.float32))


def test_split_keeps_the_jacobian_sparse(monkeypatch):
    """test/test_layers.py:642-651: both halves keep one stored row."""
    cpu_kernels.install(monkeypatch)
    x = np.random.default_rng(0).normal(size=16).astype(np.float32)
    a, b = folx_amd.forward_laplacian(lambda z: fnp.split(z, 2), 1)(x)
    assert tuple(a.jacobian.data.shape) == (1, 1, 8) and tuple(b.jacobian.data.shape) == (1, 1, 8)   # (rows, walkers, 8)
    np.testing.assert_array_equal(a.jacobian.x0_idx, np.arange(8)[None])
    np.testing.assert_array_equal(b.jacobian.x0_idx, np.arange(8, 16)[None])


def test_conversion_to_float_keeps_the_triplet_and_to_integers_drops_it(monkeypatch):
    """test/test_layers.py:531-563: float targets give a triplet (float32 is the one arithmetic type here), integer and
    boolean targets a plain array without derivatives."""
    cpu_kernels.install(monkeypatch)
    x = np.random.default_rng(1).normal(size=16).astype(np.float32)
    for dtype in (np.float16, np.float32, np.float64):
        y = folx_amd.forward_laplacian(lambda z: fnp.astype(z, dtype), 0)(x)
        assert isinstance(y, folx_amd.FwdLaplArray) and y.x.dtype == torch.float32
        np.testing.assert_array_equal(y.x[0].numpy(), x)
    for dtype in (np.bool_, np.int8, np.int16, np.int32, np.int64, np.uint8, np.uint16, np.uint32, np.uint64):
        y = folx_amd.forward_laplacian(lambda z: fnp.astype(z, dtype), 0)(x)
        assert not isinstance(y, folx_amd.FwdLaplArray)
        want = (x != 0) if dtype is np.bool_ else np.trunc(x)
        np.testing.assert_array_equal(np.asarray(getattr(y, 'data', y), dtype=np.float64).reshape(-1), want.astype(np.float64))


def _multi_output_functions():
    """test/test_layers.py:565-640: functions with two outputs -- by a derivative rule of the caller's own
    (``custom_jvp``) and by the generic rule applied element by element (``in_axes=()``)."""
    @folx_amd.custom_jvp
    def sincos(x):
        return torch.sin(x), torch.cos(x)

    @sincos.defjvp
    def sincos_jvp(primals, tangents):
        (x,), (dx,) = primals, tangents
        return sincos(x), (torch.cos(x) * dx, -torch.sin(x) * dx)

    @folx_amd.custom_jvp
    def sumdiff(a, b):
        return a + b, a - b

    @sumdiff.defjvp
    def sumdiff_jvp(primals, tangents):
        (a, b), (da, db) = primals, tangents
        return sumdiff(a, b), (da + db, da - db)

    sincos_el = folx_amd.wrap_forward_laplacian(lambda x: (torch.sin(x), torch.cos(x)), in_axes=(), name='sincos_elemwise')
    sumdiff_el = folx_amd.wrap_forward_laplacian(lambda a, b: (a + b, a - b), in_axes=(), name='sumdiff_elemwise')
    t_sumdiff = lambda z: (torch.sin(z) + torch.cos(z), torch.sin(z) - torch.cos(z))     # noqa: E731
    t_sincos = lambda z: (torch.sin(z), torch.cos(z))                                    # noqa: E731
    return {
        'single_arg': (lambda x: sincos(x), t_sincos),
        'multi_arg': (lambda x: sumdiff(fnp.sin(x), fnp.cos(x)), t_sumdiff),
        'single_arg_elemwise': (lambda x: fnp.call('sincos_elemwise', x), t_sincos),
        'multi_arg_elemwise': (lambda x: fnp.call('sumdiff_elemwise', fnp.sin(x), fnp.cos(x)), t_sumdiff),
    }, {'sincos_elemwise': sincos_el, 'sumdiff_elemwise': sumdiff_el}


def _check_multi_output(device):
    fns, rules = _multi_output_functions()
    for n, r in rules.items():
        folx_amd.register_function(n, r)
    try:
        x = np.random.default_rng(8).normal(size=8).astype(np.float32)
        xin = torch.as_tensor(x).to(device) if device != 'cpu' else x
        for name, (f, g) in fns.items():
            for thr in (0, x.size):
                y = folx_amd.forward_laplacian(f, thr)(xin)
                assert len(y) == 2
                for i, y_i in enumerate(y):
                    wy, wJ, wL = brute_force_single(lambda z, i=i: g(z)[i], x.astype(np.float64))
                    np.testing.assert_allclose(y_i.x[0].cpu().numpy(), wy, rtol=2e-5, atol=2e-6, err_msg=name)
                    np.testing.assert_allclose(y_i.jacobian.dense_array[:, 0].cpu().numpy(), wJ, rtol=2e-5, atol=2e-6, err_msg=name)
                    np.testing.assert_allclose(y_i.laplacian[0].cpu().numpy(), wL, rtol=1e-4, atol=1e-5, err_msg=name)
    finally:
        for n in rules:
            folx_amd.deregister_function(n)


def test_multi_output_functions(monkeypatch):
    cpu_kernels.install(monkeypatch)
    _check_multi_output('cpu')


@pytest.mark.gpu
def test_multi_output_functions_on_the_gpu():
    _check_multi_output('cuda')


def _grad_inside(z):
    """test/test_layers.py:684-693: a gradient taken INSIDE the function (its trace holds the accumulation of
    cotangents, ``add_any`` in jax)."""
    return torch.func.grad(lambda y: torch.sin(y).sum() + (y ** 2).sum())(z) * z


def test_function_with_a_gradient_inside_through_the_traced_front_door(monkeypatch):
    cpu_kernels.install(monkeypatch)
    x = np.random.default_rng(9).normal(size=6).astype(np.float32)
    wy, wJ, wL = brute_force_single(lambda z: (torch.cos(z) + 2 * z) * z, x.astype(np.float64))
    for thr in (0, x.size):
        y = folx_amd.forward_laplacian_torch(_grad_inside, thr)(x)
        np.testing.assert_allclose(y.x[0].numpy(), wy, rtol=2e-5, atol=2e-6)
        np.testing.assert_allclose(y.jacobian.dense_array[:, 0].numpy(), wJ, rtol=2e-5, atol=2e-6)
        np.testing.assert_allclose(y.laplacian[0].numpy(), wL, rtol=1e-4, atol=1e-5)
        assert y.jacobian.weak == (thr > 0)       # elementwise throughout: one stored row per entry

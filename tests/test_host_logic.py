"""Host logic of the product (rule composition, mask propagation, index tables) on CPU
stand-ins for the kernels: results must equal the dense oracle and brute-force AD, and
sparse / dense runs of the same model must agree."""

import numpy as np
import pytest
import torch

import cpu_kernels
from bruteforce import brute_force, plain
from oracle import backend as ob

import folx_amd
from folx_amd import numpy as fnp
from folx_amd import workloads as wl


@pytest.fixture(autouse=True)
def _cpu(monkeypatch):
    cpu_kernels.install(monkeypatch)
    from folx_amd import sparse_ops

    sparse_ops.clear_caches()


def run_product(fn, x, thr):
    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
    return out


def triplet_np(out):
    return (out.x.numpy().astype(np.float64), out.jacobian.dense_array.numpy().astype(np.float64),
            out.laplacian.numpy().astype(np.float64))


def check_against_oracle(fn, x, thr, rtol=2e-4, atol=2e-5):
    got = triplet_np(run_product(fn, x, thr))
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    P = ref.J.shape[0]
    J = got[1]
    if J.shape[0] < P:  # trailing inputs nothing depends on (dense_array is max_n + 1 rows)
        J = np.concatenate([J, np.zeros((P - J.shape[0], *J.shape[1:]))], 0)
    np.testing.assert_allclose(got[0], ref.x, rtol=rtol, atol=atol)
    np.testing.assert_allclose(J, ref.J, rtol=rtol, atol=atol)
    np.testing.assert_allclose(got[2], ref.lap, rtol=rtol, atol=atol)
    return got


@pytest.mark.parametrize('thr', [0, 4, 3, 100])
def test_nodewise_mlp(thr):
    """README example in miniature; thr=4 keeps k=4 rows, thr=3 falls back to dense."""
    params = wl.mlp_params(seed=0, in_dim=4, width=8, n_hidden=3)
    x = np.random.default_rng(0).normal(size=(3, 6, 4)).astype(np.float32)
    fn = lambda xp, t: wl.mlp_forward(params, t, xp)
    check_against_oracle(fn, x, thr)


def test_nodewise_mlp_sparsity_pattern():
    """k stays 4 through the hidden layers (node-wise MLP, README.md:41-70) and the final
    sum switches to the dense Jacobian (400 > threshold)."""
    params = wl.mlp_params(seed=0, in_dim=4, width=8, n_hidden=2)
    x = np.random.default_rng(0).normal(size=(2, 5, 4)).astype(np.float32)
    seen = []

    def fn(t):
        h = t
        for W, b in params[:-1]:
            h = fnp.silu(fnp.dot(h, W, b))
            seen.append(h.jacobian)
        h = fnp.dot(h, *params[-1])
        seen.append(h.jacobian)
        return fnp.sum(h)

    out = folx_amd.vmap(folx_amd.forward_laplacian(fn, 4))(x)
    for jac in seen:
        assert jac.weak and jac.data.shape[0] == 4
        # node m depends on inputs 4m .. 4m+3, ascending, identical across features
        want = (4 * np.arange(5)[None, :, None] + np.arange(4)[:, None, None])
        np.testing.assert_array_equal(jac.x0_idx, np.broadcast_to(want, jac.x0_idx.shape))
    assert not out.jacobian.weak and out.jacobian.data.shape[0] == 20


BINARY_FNS = {
    'same_mask_mul': lambda xp, x: xp.multiply(xp.tanh(x), xp.exp(x)),
    'same_mask_div': lambda xp, x: xp.divide(xp.sin(x), xp.add(xp.square(x), 1.0)),
    'diff_mask_sub': lambda xp, x: xp.subtract(xp.expand_dims(x, 1), xp.expand_dims(xp.tanh(x), 0)),
    'diff_mask_mul': lambda xp, x: xp.multiply(xp.expand_dims(x, 1), xp.expand_dims(xp.sin(x), 0)),
    'diff_mask_div': lambda xp, x: xp.divide(xp.expand_dims(x, 1), xp.add(xp.expand_dims(xp.square(x), 0), 1.0)),
    'dup_then_unary': lambda xp, x: xp.tanh(xp.add(xp.expand_dims(x, 1), xp.expand_dims(x, 0))),
    'const_ops': lambda xp, x: xp.divide(2.0, xp.add(xp.multiply(xp.subtract(1.5, x), np.arange(1, 4.0)), 7.0)),
}


@pytest.mark.parametrize('name', sorted(BINARY_FNS))
@pytest.mark.parametrize('thr', [0, 2, 6, 100])
def test_binary_rules(name, thr):
    x = np.random.default_rng(1).normal(size=(2, 4, 3)).astype(np.float32)
    got = check_against_oracle(BINARY_FNS[name], x, thr)
    by, bJ, bL = brute_force(lambda t: BINARY_FNS[name](plain, t), x.astype(np.float64))
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-5)


def test_duplicate_mask_layout_follows_reference():
    """x[:, None] + x[None, :] concatenates the two one-row masks (folx/jvp.py:294-317):
    k = 2 with the diagonal listing the same input twice; the following tanh keeps the
    rows (folx/jvp.py:262-272) and takes its Hessian term on the unique frame."""
    x = np.random.default_rng(2).normal(size=(1, 3)).astype(np.float32)

    def fn(t):
        s = fnp.add(fnp.expand_dims(t, 1), fnp.expand_dims(t, 0))
        assert s.jacobian.x0_idx.shape == (2, 3, 3)
        np.testing.assert_array_equal(s.jacobian.x0_idx[:, 1, 1], [1, 1])
        return fnp.tanh(s)

    out = folx_amd.vmap(folx_amd.forward_laplacian(fn, 4))(x)
    assert out.jacobian.x0_idx.shape == (2, 3, 3)
    xs = x[0].astype(np.float64)
    s = xs[:, None] + xs[None, :]
    t = np.tanh(s)
    cnt = np.where(np.eye(3, dtype=bool), 4.0, 2.0)  # |grad s|^2: (2)^2 on the diagonal, 1 + 1 off it
    np.testing.assert_allclose(out.laplacian[0].numpy(), -2 * t * (1 - t * t) * cnt, rtol=1e-5, atol=1e-6)


REDUCE_FNS = {
    'sum_all': lambda xp, x: xp.sum(xp.tanh(x)),
    'sum_last': lambda xp, x: xp.sum(xp.square(x), axis=-1),
    'sum_first_keep': lambda xp, x: xp.sum(xp.exp(x), axis=0, keepdims=True),
    'mean_mid': lambda xp, x: xp.mean(xp.sin(xp.expand_dims(x, 1) * 1.0 if xp is plain else xp.multiply(xp.expand_dims(x, 1), 1.0)), axis=1),
    'dist': lambda xp, x: xp.sqrt(xp.sum(xp.square(xp.subtract(xp.expand_dims(x, 1), np.arange(6.0).reshape(2, 3))), axis=-1)),
}


@pytest.mark.parametrize('name', sorted(REDUCE_FNS))
@pytest.mark.parametrize('thr', [0, 3, 12])
def test_reductions(name, thr):
    x = np.random.default_rng(3).normal(size=(2, 4, 3)).astype(np.float32)
    check_against_oracle(REDUCE_FNS[name], x, thr)


def test_indexing_rules():
    R = np.random.default_rng(4).normal(size=(2, 3))

    def fn(xp, r):
        d = xp.subtract(xp.expand_dims(r, 1), R)
        dist = xp.sqrt(xp.sum(xp.square(d), axis=-1))
        f = xp.concatenate([xp.reshape(d, (4, 6)), dist, np.ones((4, 1))], axis=-1)
        f = xp.transpose(f, (1, 0))
        return xp.getitem(f, (slice(1, 8),))

    x = np.random.default_rng(5).normal(size=(2, 4, 3)).astype(np.float32)
    for thr in (0, 3, 6):
        check_against_oracle(fn, x, thr)
    # constants keep sparsity (test/test_layers.py:763-776): k stays 3 after the concat
    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), 6))(x)
    assert out.jacobian.weak and out.jacobian.data.shape[0] == 3


def test_operator_and_single_sample_api():
    """README.md:22-33: f(x) = sum x^2 at arange(3) -> 5, [0, 2, 4], 6."""
    f = lambda x: fnp.sum(fnp.square(x))
    for thr in (0, 3):
        res = folx_amd.forward_laplacian(f, thr)(np.arange(3, dtype=np.float32))
        assert float(res.x[0]) == 5.0
        np.testing.assert_allclose(res.jacobian.dense_array[:, 0].numpy(), [0, 2, 4])
        assert float(res.laplacian[0]) == 6.0
        lap, jac = folx_amd.ForwardLaplacianOperator(thr)(f)(np.arange(3, dtype=np.float32))
        assert float(lap) == 6.0 and jac.shape == (3,)


def test_weights_argument():
    f = lambda x: fnp.sum(fnp.exp(x))
    x = np.array([[0.1, -0.3, 0.7]], dtype=np.float32)
    w = np.array([1.0, 0.0, 2.0], dtype=np.float32)
    for thr in (0, 3):
        res = folx_amd.forward_laplacian(f, thr).batched(x, weights=w)
        np.testing.assert_allclose(res.jacobian.dense_array[:, 0].numpy(), np.exp(x[0]) * w, rtol=1e-6)
        np.testing.assert_allclose(float(res.laplacian[0]), (np.exp(x[0]) * w * w).sum(), rtol=1e-6)


def test_batched_vmap_chunks():
    f = lambda x: fnp.sum(fnp.tanh(x))
    x = np.random.default_rng(6).normal(size=(7, 5)).astype(np.float32)
    full = folx_amd.vmap(folx_amd.forward_laplacian(f, 0))(x)
    for mb in (2, 3, 7, 10):
        part = folx_amd.batched_vmap(folx_amd.forward_laplacian(f, 0), mb)(x)
        np.testing.assert_allclose(part.x.numpy(), full.x.numpy())
        np.testing.assert_allclose(part.laplacian.numpy(), full.laplacian.numpy())
        np.testing.assert_allclose(part.jacobian.data.numpy(), full.jacobian.data.numpy())


def test_batched_vmap_in_axes():
    """An argument is cut into chunks only when ``in_axes`` says it has a walker axis (folx/vmap.py:11-30):
    an array with B leading entries under ``None`` is shown whole to every walker, whatever the chunk size;
    an int other than 0 names the walker axis."""
    rng = np.random.default_rng(8)
    B = 5
    x = rng.normal(size=(B, 4)).astype(np.float32)
    c = rng.normal(size=(B, 4)).astype(np.float32)      # a second input that happens to have B rows, no walker axis
    f = lambda u, v: fnp.sum(fnp.multiply(fnp.tanh(u), fnp.sum(fnp.sin(v), axis=0)))
    fl = folx_amd.forward_laplacian(f, 0)
    full = folx_amd.batched_vmap(fl, 100, in_axes=(0, None))(x, c)
    ref = folx_amd.vmap(fl)(x, np.broadcast_to(c[None], (B, B, 4)))
    np.testing.assert_allclose(full.laplacian.numpy(), ref.laplacian.numpy(), rtol=1e-6)
    for mb in (2, 3):
        part = folx_amd.batched_vmap(fl, mb, in_axes=(0, None))(x, c)
        np.testing.assert_allclose(part.x.numpy(), full.x.numpy(), rtol=1e-6)
        np.testing.assert_allclose(part.laplacian.numpy(), full.laplacian.numpy(), rtol=1e-6)
        np.testing.assert_allclose(part.jacobian.dense_array.numpy(), full.jacobian.dense_array.numpy(), rtol=1e-6)
    g = folx_amd.forward_laplacian(lambda u: fnp.sum(fnp.tanh(u)), 0)
    a = folx_amd.batched_vmap(g, 2, in_axes=1)(np.ascontiguousarray(x.T))
    b = folx_amd.vmap(g)(x)
    np.testing.assert_allclose(a.laplacian.numpy(), b.laplacian.numpy(), rtol=1e-6)
    with pytest.raises(NotImplementedError):
        folx_amd.batched_vmap(g, 2, out_axes=1)


def test_batched_vmap_uneven_multiple_arguments_and_nested():
    """The reference's own cases (test/test_vmap.py:23-66): a batch that the chunk size does not divide, two
    mapped arguments, and two nested levels ``batched_vmap(batched_vmap(f, m, (0, None)), m, (None, 0))`` whose
    result carries both axes, for chunk sizes 10, 5 and 1; here ``f`` is the Laplacian operator of
    ``vdot(sin x, cos y)``, whose Laplacian is ``-2 vdot(sin x, cos y)``."""
    rng = np.random.default_rng(42)
    f = lambda u, v: fnp.sum(fnp.multiply(fnp.sin(u), fnp.cos(v)))
    fl = folx_amd.forward_laplacian(f, 0)

    class op:  # Laplacian and gradient as tensors with the walker axis in front (the operators take one argument)
        @staticmethod
        def batched(*args):
            out = fl.batched(*args)
            return out.laplacian, out.jacobian.dense_array.movedim(0, -1)
    a21, b21 = rng.normal(size=(21, 3)).astype(np.float32), rng.normal(size=(21, 3)).astype(np.float32)
    want = -2.0 * (np.sin(a21.astype(np.float64)) * np.cos(b21.astype(np.float64))).sum(-1)
    for mb in (10, 5, 1):
        lap, jac = folx_amd.batched_vmap(op, mb)(a21, b21)
        assert tuple(lap.shape) == (21,) and tuple(jac.shape) == (21, 6)
        np.testing.assert_allclose(lap.numpy(), want, rtol=1e-5, atol=1e-6)
    a, b = a21[:10], b21[:7]
    want2 = -2.0 * np.einsum('ik,jk->ji', np.sin(a.astype(np.float64)), np.cos(b.astype(np.float64)))  # [j over b][i over a]
    for mb in (10, 5, 1):
        lap, jac = folx_amd.batched_vmap(folx_amd.batched_vmap(op, mb, in_axes=(0, None)), mb, in_axes=(None, 0))(a, b)
        assert tuple(lap.shape) == (7, 10) and tuple(jac.shape) == (7, 10, 6)
        np.testing.assert_allclose(lap.numpy(), want2, rtol=1e-5, atol=1e-6)
    # the outer level may also be the plain vmap
    lap, _ = folx_amd.vmap(folx_amd.batched_vmap(op, 4, in_axes=(0, None)))(
        np.broadcast_to(a[None], (7, 10, 3)).copy(), b)
    np.testing.assert_allclose(lap.numpy(), want2, rtol=1e-5, atol=1e-6)
    with pytest.raises(NotImplementedError):  # a triplet has one walker axis
        folx_amd.vmap(folx_amd.batched_vmap(folx_amd.forward_laplacian(f, 0), 4, in_axes=(0, None)))(
            np.broadcast_to(a[None], (7, 10, 3)).copy(), b)


def test_constant_cache_keeps_scalars_and_one_element_vectors_apart():
    """Constants are cached by content AND shape: a scalar 0.0 and ``zeros(1)`` have the same bytes (and
    ``numpy.ascontiguousarray`` gives both the shape (1,)), but not the same entry."""
    from folx_amd import sparse_ops as so

    so.clear_caches()
    cpu = torch.device('cpu')
    s = so.device_const(np.float32(0.25), cpu)
    v = so.device_const(np.full((1,), 0.25, dtype=np.float32), cpu)
    m = so.device_const(np.full((1, 1), 0.25, dtype=np.float32), cpu)
    assert tuple(s.shape) == () and tuple(v.shape) == (1,) and tuple(m.shape) == (1, 1)
    assert so.device_const(np.float32(0.25), cpu) is s and so.device_const(np.full((1,), 0.25, dtype=np.float32), cpu) is v


def test_register_function_plugs_in():
    calls = []

    def my_tanh(args, kwargs, sparsity_threshold):
        calls.append(sparsity_threshold)
        return folx_amd.wrapped_functions._unary_rule('tanh')(args, kwargs, sparsity_threshold)

    old = folx_amd.get_laplacian('tanh')
    folx_amd.register_function('tanh', my_tanh)
    try:
        folx_amd.forward_laplacian(lambda x: fnp.tanh(x), 5)(np.zeros(2, np.float32))
    finally:
        folx_amd.register_function('tanh', old)
    assert calls == [5]
    folx_amd.register_function('my_op', my_tanh)
    assert folx_amd.is_registered('my_op')
    folx_amd.deregister_function('my_op')
    assert not folx_amd.is_registered('my_op')
    with pytest.raises(KeyError):
        folx_amd.get_laplacian('no_such_primitive', wrap_if_missing=True)


SMALL_PSI = wl.PsiFormerConfig(n_elec=4, n_nuc=2, n_layers=2, n_heads=2, head_dim=4, width=8, mlp_width=8, n_det=2)


@pytest.mark.parametrize('thr', [0, 6])
def test_psiformer_small_vs_oracle_and_bruteforce(thr):
    p = wl.psiformer_params(SMALL_PSI)
    x = wl.sample_electrons(2, SMALL_PSI.n_elec, 1.0, seed=3)
    fn = lambda xp, t: wl.psiformer_forward(p, t, xp)
    got = check_against_oracle(fn, x, thr, rtol=5e-4, atol=5e-5)
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    np.testing.assert_allclose(ref.x, by, rtol=1e-8)
    np.testing.assert_allclose(ref.J, bJ, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(ref.lap, bL, rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(got[2], bL, rtol=5e-4, atol=5e-5)


def test_psiformer_sparse_stage_keeps_three_rows():
    """Before the first attention layer every per-electron quantity depends on that
    electron's three coordinates only: k = 3 with thr = 6 (README.md:72)."""
    p = wl.psiformer_params(SMALL_PSI)
    x = wl.sample_electrons(2, SMALL_PSI.n_elec, 1.0, seed=3)
    seen = {}

    def fn(r):
        d, dist = wl.electron_nuclear_features(fnp, r, p.nuclei)
        seen['d'], seen['dist'] = d.jacobian, dist.jacobian
        feats = fnp.concatenate([fnp.reshape(d, (4, 6)), dist, p.spin], axis=-1)
        h = fnp.dot(feats, p.w_in)
        seen['h'] = h.jacobian
        hn = wl.layer_norm(fnp, h, p.layers[0]['ln1_g'], p.layers[0]['ln1_b'], 1e-5)
        seen['ln'] = hn.jacobian
        return fnp.sum(hn)

    folx_amd.vmap(folx_amd.forward_laplacian(fn, 6))(x)
    assert seen['d'].x0_idx.shape[0] == 1 and seen['dist'].x0_idx.shape[0] == 3
    for key in ('h', 'ln'):
        jac = seen[key]
        assert jac.weak and jac.x0_idx.shape[0] == 3
        want = 3 * np.arange(4)[None, :, None] + np.arange(3)[:, None, None]
        np.testing.assert_array_equal(jac.x0_idx, np.broadcast_to(want, jac.x0_idx.shape))


@pytest.mark.parametrize('thr', [0, 6])
def test_layer_norm_rule_fused_equals_primitive_chain(thr):
    g, b = np.linspace(0.5, 1.5, 8), np.linspace(-1, 1, 8)
    W = np.random.default_rng(7).normal(size=(3, 8))
    x = np.random.default_rng(8).normal(size=(2, 4, 3)).astype(np.float32)
    fused = lambda xp, t: xp.layer_norm(xp.dot(t, W), g, b, 1e-5)
    chain = lambda xp, t: wl.layer_norm_primitives(xp, xp.dot(t, W), g, b, 1e-5)
    a = check_against_oracle(fused, x, thr)
    c = triplet_np(run_product(chain, x, thr))
    for u, v in zip(a, c):
        np.testing.assert_allclose(u, v, rtol=2e-4, atol=2e-5)
    # sparse input whose mask varies along the normalised axis: falls back to the chain
    varying = lambda xp, t: xp.layer_norm(xp.reshape(t, (3, 4)), None, None, 1e-5)
    check_against_oracle(varying, x, thr)
    out = run_product(fused, x, 6)
    assert out.jacobian.weak and out.jacobian.x0_idx.shape[0] == 3


MATMUL_FNS = {
    'mat_mat': lambda xp, x: xp.matmul(xp.tanh(x), xp.swapaxes(xp.sin(x), -1, -2)),        # (4,3)@(3,4)
    'attn_like': lambda xp, x: xp.matmul(xp.exp(xp.multiply(xp.matmul(x, xp.swapaxes(x, -1, -2)), 0.1)), x),
    'vec_mat': lambda xp, x: xp.matmul(xp.getitem(x, (0,)), xp.swapaxes(xp.cos(x), -1, -2)),  # (3,)@(3,4)
    'const_left': lambda xp, x: xp.matmul(np.arange(8.0).reshape(2, 4) / 8, xp.tanh(x)),      # (2,4)@(4,3)
    # test/test_layers.py:141-171: attention and a rectangular product of two functions of x
    'attn': lambda xp, x: xp.matmul(xp.exp(xp.matmul(xp.multiply(x, 0.3), xp.swapaxes(x, -2, -1))), x),
    'rect': lambda xp, x: xp.matmul(xp.sin(x), xp.cos(xp.swapaxes(x, -2, -1))),
    # test/test_layers.py:173-206: einsums with degenerate broadcast dimensions
    'ein_n1': lambda xp, x: xp.einsum('nk,mk->nm', x, xp.sin(xp.getitem(x, (slice(0, 1),)))),
    'ein_1n': lambda xp, x: xp.einsum('nk,mk->nm', xp.getitem(x, (slice(0, 1),)), xp.sin(x)),
    'ein_vec': lambda xp, x: xp.einsum('k,mk->m', xp.getitem(x, (0,)), xp.sin(xp.getitem(x, (slice(0, 3),)))),
    'ein_mpnn': lambda xp, x: xp.einsum('ijh,jh->ih', xp.sin(xp.multiply(xp.expand_dims(x, 1), xp.expand_dims(x, 0))),
                                        xp.cos(x)),
    # test/test_composite.py:45-83: softmax attention from three projections, summed
    'softmax_attn': lambda xp, x: xp.sum(xp.matmul(
        xp.softmax(xp.matmul(xp.dot(x, _ATT_W[0]), xp.swapaxes(xp.dot(x, _ATT_W[1]), -1, -2)), axis=-1),
        xp.dot(x, _ATT_W[2]))),
}
_ATT_W = [np.random.default_rng(40 + i).normal(size=(3, 8)).astype(np.float32) / 2 for i in range(3)]


from one_constant_cases import ONE_CONSTANT_FNS  # noqa: E402
from size_limit_cases import BIG_MATRIX_FNS  # noqa: E402


@pytest.mark.parametrize('name', sorted(ONE_CONSTANT_FNS))
@pytest.mark.parametrize('thr', [0, 12])
def test_dot_general_with_one_constant_operand(name, thr):
    """One operand with derivatives against a constant of any rank, on either side, with any
    contracted and batch axes (``_dot_general_one_constant``, folx/wrapped_functions.py:71-171; the
    real half of test/test_layers.py:119-139 is 'matmul_vec' / 'vec_matmul' / the 2-D cases of
    MATMUL_FNS): dense (threshold 0) and sparse (threshold = number of inputs)."""
    x = np.random.default_rng(9).normal(size=(2, 4, 3)).astype(np.float32)
    fn = ONE_CONSTANT_FNS[name]
    got = check_against_oracle(fn, x, thr)
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
    np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[1], bJ[: got[1].shape[0]], rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-5)


def test_batched_constant_product_keeps_sparse_rows():
    """Per-position weights applied to a node-wise feature keep one Jacobian row per input
    coordinate of the node (the mask is constant along the contracted axis only after the union
    over it: 3 rows), where a dense run has all 12."""
    x = np.random.default_rng(9).normal(size=(2, 4, 3)).astype(np.float32)
    out = run_product(ONE_CONSTANT_FNS['einsum_heads'], x, 12)
    assert out.jacobian.weak and out.jacobian.x0_idx.shape[0] == 3
    dense = run_product(ONE_CONSTANT_FNS['einsum_heads'], x, 0)
    assert not dense.jacobian.weak
    np.testing.assert_allclose(out.jacobian.dense_array.numpy(), dense.jacobian.dense_array.numpy(), rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize('name', sorted(MATMUL_FNS))
@pytest.mark.parametrize('thr', [0, 12])
def test_two_operand_matmul(name, thr):
    """test/test_layers.py:141-171 (matmul with both operands carrying Jacobians)."""
    x = np.random.default_rng(9).normal(size=(2, 4, 3)).astype(np.float32)
    got = check_against_oracle(MATMUL_FNS[name], x, thr)
    by, bJ, bL = brute_force(lambda t: MATMUL_FNS[name](plain, t), x.astype(np.float64))
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize('thr', [0, 9])
def test_det_rule(thr):
    """test/test_layers.py:424-444."""
    W = np.random.default_rng(10).normal(size=(5, 9)) / 2
    fn = lambda xp, x: xp.det(xp.reshape(xp.tanh(xp.dot(x, W)), (3, 3)))
    x = np.random.default_rng(11).normal(size=(3, 5)).astype(np.float32)
    got = check_against_oracle(fn, x, thr)
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
    np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-5)


SMALL_FERMI = wl.FermiNetConfig(n_elec=4, n_nuc=2, n_layers=3, w1=8, w2=4, n_det=2)


@pytest.mark.parametrize('thr', [0, 6])
def test_ferminet_small_vs_oracle_and_bruteforce(thr):
    p = wl.ferminet_params(SMALL_FERMI)
    x = wl.sample_electrons(2, SMALL_FERMI.n_elec, 1.0, seed=4)
    fn = lambda xp, t: wl.ferminet_forward(p, t, xp)
    got = check_against_oracle(fn, x, thr, rtol=5e-4, atol=5e-5)
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    np.testing.assert_allclose(ref.x, by, rtol=1e-8)
    np.testing.assert_allclose(ref.J, bJ, rtol=1e-6, atol=1e-9)
    np.testing.assert_allclose(ref.lap, bL, rtol=1e-6, atol=1e-8)
    np.testing.assert_allclose(got[2], bL, rtol=5e-4, atol=5e-5)


def test_ferminet_pair_stream_stays_sparse():
    """The pair stream depends on six coordinates per pair: k = 6 with thr = 6, through
    the tanh layers and the residual adds (README.md:72)."""
    p = wl.ferminet_params(SMALL_FERMI)
    x = wl.sample_electrons(2, SMALL_FERMI.n_elec, 1.0, seed=4)
    seen = {}

    def fn(r):
        rij = fnp.subtract(fnp.expand_dims(r, 1), fnp.expand_dims(r, 0))
        seen['rij'] = rij.jacobian
        r2 = fnp.add(fnp.sum(fnp.square(rij), axis=-1), p.eye)
        seen['r2'] = r2.jacobian
        rn = fnp.multiply(fnp.sqrt(r2), 1.0 - p.eye)
        g = fnp.concatenate([rij, fnp.expand_dims(rn, 2)], axis=-1)
        seen['g'] = g.jacobian
        g2 = fnp.tanh(fnp.dot(g, p.layers[0]['w'], p.layers[0]['c']))
        seen['g2'] = g2.jacobian
        return fnp.sum(g2)

    folx_amd.vmap(folx_amd.forward_laplacian(fn, 6))(x)
    assert seen['rij'].x0_idx.shape[0] == 2          # rows of r_i and of r_j
    assert seen['r2'].x0_idx.shape[0] == 6           # union over xyz of both electrons
    assert seen['g'].x0_idx.shape[0] == 6 and seen['g2'].x0_idx.shape[0] == 6
    i, j = 1, 3
    assert sorted(int(v) for v in seen['g2'].x0_idx[:, i, j, 0]) == [3, 4, 5, 9, 10, 11]
    # a diagonal pair depends on three coordinates only
    assert sorted(set(int(v) for v in seen['g2'].x0_idx[:, 2, 2, 0] if v >= 0)) == [6, 7, 8]


@pytest.mark.parametrize('thr', [0, 3, 100])
def test_dot_row_slice(thr):
    """``dot(h, W, row_slice=...)`` equals slicing first, for dense Jacobians, for sparse
    ones that pass through unchanged and for sparse ones that need re-indexing."""
    rng = np.random.default_rng(9)
    W1 = rng.normal(size=(3, 8)).astype(np.float32)
    W2 = rng.normal(size=(8, 5)).astype(np.float32)
    x = rng.normal(size=(2, 6, 3)).astype(np.float32)

    def fn(xp, t):
        h = xp.tanh(xp.dot(t, W1))                       # (6, 8), k = 3 per node
        a = xp.dot(h, W2, row_slice=(1, 4))              # rows pass through
        b = xp.dot(xp.transpose(h, (1, 0)), W2[:6, :], row_slice=(2, 7))  # contraction over nodes: re-indexed
        return xp.add(xp.sum(a), xp.sum(b))

    check_against_oracle(fn, x, thr)


@pytest.mark.parametrize('thr', [0, 3, 100])
def test_dot_act(thr):
    """``dot(h, W, b, act=...)`` equals the dense rule followed by the elementwise rule: on the
    fused kernel's shapes (dense and sparse rows), past them (K not a multiple of 4), with a
    union over the contracted axis and with a residual added after the activation."""
    rng = np.random.default_rng(10)
    W0 = rng.normal(size=(3, 8)).astype(np.float32)
    W1 = rng.normal(size=(8, 8)).astype(np.float32) / 3
    b1 = rng.normal(size=(8,)).astype(np.float32)
    W2 = rng.normal(size=(6, 4)).astype(np.float32) / 3
    W3 = rng.normal(size=(4, 5)).astype(np.float32) / 2
    x = rng.normal(size=(2, 6, 3)).astype(np.float32)

    def fn(xp, t):
        h = xp.dot(t, W0, act='tanh')                               # K = 3: two rules
        h = xp.dot(h, W1, b1, act='silu', residual=h)               # fused, rows pass through
        g = xp.dot(xp.transpose(h, (1, 0)), W2, act='sigmoid')      # contraction over nodes: union frame
        return xp.add(xp.sum(xp.dot(g, W3, act='softplus')), xp.sum(h))

    check_against_oracle(fn, x, thr)


@pytest.mark.parametrize('thr', [0, 6])
def test_dot_norm(thr, monkeypatch):
    """``dot(h, W, b, norm=..., act=...)`` equals layer_norm, dense and elementwise rules one
    after the other: through the fused rule on wide layers over dense Jacobians (with and
    without an activation, with a residual), and through the three rules on sparse Jacobians
    and on narrow layers."""
    from folx_amd import kernels as K

    calls = []
    orig = K.norm_dense
    monkeypatch.setattr(K, 'norm_dense', lambda *a: (calls.append(a[0]), orig(*a))[1])
    rng = np.random.default_rng(12)
    W0 = rng.normal(size=(3, 16)).astype(np.float32)
    g0, b0 = (1 + 0.2 * rng.normal(size=16)).astype(np.float32), (0.2 * rng.normal(size=16)).astype(np.float32)
    W1 = rng.normal(size=(16, 132)).astype(np.float32) / 4
    c1 = rng.normal(size=(132,)).astype(np.float32)
    W2 = rng.normal(size=(132, 16)).astype(np.float32) / 11
    W3 = rng.normal(size=(16, 136)).astype(np.float32) / 4
    W4 = rng.normal(size=(16, 8)).astype(np.float32) / 4
    x = rng.normal(size=(2, 10, 3)).astype(np.float32)  # 30 Jacobian rows: one well-filled group of 32

    def fn(xp, t):
        h = xp.dot(t, W0)                                                    # sparse rows at thr 6
        a = xp.dot(h, W1, c1, norm=(g0, b0, 1e-5), act='tanh')               # sparse: three rules; dense: fused
        h = xp.add(xp.dot(a, W2), xp.mean(h, axis=0, keepdims=True))         # mixes electrons: dense from here on
        u = xp.dot(h, W3, norm=(g0, None, 1e-5))                             # fused, no activation
        v = xp.dot(h, W3, norm=(None, None, 1e-3), act='silu', residual=u)   # fused, residual added afterwards
        w = xp.dot(h, W4, norm=(g0, b0, 1e-5), act='sin')                    # narrow: layer_norm, then dense + act
        hn = xp.layer_norm(h, g0, b0, 1e-5, lazy=True)                       # a handle that only dot consumes
        s = xp.add(xp.dot(hn, W3, act='tanh'), xp.dot(hn, W3))               # fused twice, never evaluated
        t = xp.add(xp.dot(hn, W4), xp.dot(hn, W4, act='cos'))                # narrow: evaluated once for both
        return xp.add(xp.add(xp.sum(v), xp.sum(w)), xp.add(xp.sum(s), xp.sum(t)))

    from folx_amd import wrapped_functions as wf

    lns = []
    orig_ln = wf.layer_norm_rule
    monkeypatch.setattr(wf, 'layer_norm_rule', lambda *a: (lns.append(1), orig_ln(*a))[1])
    check_against_oracle(fn, x, thr)
    assert calls == (['tanh', None, 'silu', 'tanh', None] if thr == 0 else [None, 'silu', 'tanh', None])
    # unfused evaluations of layer_norm: the narrow product, the handle's two narrow products
    # together, and at threshold 6 the product on sparse rows
    assert len(lns) == (2 if thr == 0 else 3)


@pytest.mark.parametrize('thr', [0, 6])
def test_dot_of_lazy_concatenate(thr, monkeypatch):
    """``dot(concatenate(parts, lazy=True), W, b, act=...)`` equals the evaluated chain: read
    part by part where the fused kernel applies (widths that are multiples of 16, a wide
    layer; per-walker vectors among the parts multiplied once per walker, a sparse part densified), evaluated
    once otherwise (a narrow layer, a width of 8)."""
    from folx_amd import kernels as K

    calls = []
    orig = K.dense_act_parts
    monkeypatch.setattr(K, 'dense_act_parts', lambda *a: (calls.append((tuple(a[4]), tuple(a[5]), a[6], None if a[11] is None else tuple(a[11][1].shape))), orig(*a))[1])
    rng = np.random.default_rng(14)
    n = 10
    W0 = rng.normal(size=(3, 16)).astype(np.float32)
    Wm = rng.normal(size=(16, 32)).astype(np.float32) / 4
    W1 = rng.normal(size=(16 + 32 + 16 + 16, 132)).astype(np.float32) / 9
    b1 = rng.normal(size=(132,)).astype(np.float32)
    W2 = rng.normal(size=(16 + 16, 24)).astype(np.float32) / 6
    W3 = rng.normal(size=(16 + 8, 136)).astype(np.float32) / 5
    x = rng.normal(size=(2, n, 3)).astype(np.float32)

    def fn(xp, t):
        e = xp.dot(t, W0)                                   # (n, 16), sparse rows at thr 6
        m = xp.mean(xp.tanh(e), axis=0)                     # (16,) per walker, dense
        h = xp.tanh(xp.dot(xp.add(e, m), Wm))               # (n, 32) dense
        parts = [e, h, xp.broadcast_to(m, (n, 16), lazy=True), xp.broadcast_to(xp.square(m), (n, 16), lazy=True)]
        f = xp.concatenate(parts, axis=-1, lazy=True)
        a = xp.dot(f, W1, b1, act='tanh')                   # fused: four parts, two of them broadcast
        a = xp.dot(f, W1, b1, act='tanh', residual=a)       # again, with a dense skip connection in the epilogue
        f2 = xp.concatenate([e, xp.broadcast_to(m, (n, 16), lazy=True)], axis=-1, lazy=True)
        b = xp.dot(f2, W2, act='silu')                      # narrow layer: concatenation evaluated
        f3 = xp.concatenate([e, xp.getitem(h, (slice(None), slice(0, 8)))], axis=-1, lazy=True)
        c = xp.dot(f3, W3, act='sin', residual=None)        # a width of 8: concatenation evaluated
        return xp.add(xp.add(xp.sum(a), xp.sum(b)), xp.sum(c))

    check_against_oracle(fn, x, thr)
    # the two per-walker parts meet their rows of W once per walker (pre-activation term (P, walkers, 132));
    # the product itself reads the two per-position parts
    assert calls == [((16, 32), (False, False), n, (3 * n, 2, 132))] * 2


@pytest.mark.parametrize('thr', [0, 6])
def test_readme_fused_layer_forms(thr):
    """The layer forms the README shows (activation and skip connection in the product, lazy
    layer_norm, lazy concatenation with a windowed mean broadcast among its parts)."""
    rng = np.random.default_rng(15)
    n, n_up, d = 8, 3, 16
    W0 = rng.normal(size=(3, d)).astype(np.float32)
    W, b = rng.normal(size=(d, d)).astype(np.float32) / 4, rng.normal(size=(d,)).astype(np.float32)
    gamma, beta = (1 + 0.1 * rng.normal(size=d)).astype(np.float32), (0.1 * rng.normal(size=d)).astype(np.float32)
    Wq, Wk = (rng.normal(size=(d, d)).astype(np.float32) / 4 for _ in range(2))
    V, c = rng.normal(size=(2 * d, d)).astype(np.float32) / 5, rng.normal(size=(d,)).astype(np.float32)
    x0 = rng.normal(size=(2, n, 3)).astype(np.float32)

    def fn(xp, t):
        x = xp.dot(t, W0)
        h = xp.dot(x, W, b, act='tanh', residual=x)
        hn = xp.layer_norm(h, gamma, beta, 1e-5, lazy=True)
        q, k = xp.dot(hn, Wq), xp.dot(hn, Wk)
        f = xp.concatenate([h, xp.broadcast_to(xp.mean(h, axis=0, window=(0, n_up)), h.shape, lazy=True)], lazy=True)
        h = xp.dot(f, V, c, act='tanh', residual=h)
        return xp.add(xp.sum(xp.multiply(q, k)), xp.sum(h))

    check_against_oracle(fn, x0, thr)


def test_first_attention_layer_takes_position_sparse_path(monkeypatch):
    """q, k, v of the first PsiFormer layer still carry per-electron sparse Jacobians: the rule
    hands them to the position-sparse kernel and the result equals the densified rule."""
    import folx_amd
    from folx_amd import kernels as K
    from folx_amd import numpy as fnp
    from folx_amd import wrapped_functions as wf
    from oracle import backend as ob

    calls = []
    orig = K.mhsa_sparse
    monkeypatch.setattr(K, 'mhsa_sparse', lambda *a: (calls.append(a[9].shape), orig(*a))[1])
    rng = np.random.default_rng(13)
    n, H, d = 4, 2, 4
    Wq, Wk, Wv = (rng.normal(size=(3, H * d)).astype(np.float32) for _ in range(3))
    x = rng.normal(size=(2, n, 3)).astype(np.float32)

    def fn(xp, r):
        q = xp.reshape(xp.dot(r, Wq), (n, H, d))
        k = xp.reshape(xp.dot(r, Wk), (n, H, d))
        v = xp.reshape(xp.dot(r, Wv), (n, H, d))
        return xp.sum(xp.multi_head_self_attention(q, k, v))

    check_against_oracle(fn, x, 6)
    assert calls == [(3, n)]
    calls.clear()
    check_against_oracle(fn, x, 0)      # dense Jacobians: the ordinary kernel
    assert calls == []


@pytest.mark.parametrize('parallel', [False, True])
def test_loop_and_parallel_operators(parallel):
    """folx/operators.py:41-79: the Hessian diagonal and the gradient of a scalar function,
    one pass per coordinate (or all of them stacked along the walker axis); their sum is the
    forward Laplacian (test/test_operator.py:19-73) and they match AD in float64."""
    from bruteforce import plain

    rng = np.random.default_rng(14)
    W1 = rng.normal(size=(3, 5)).astype(np.float32)
    W2 = rng.normal(size=(5, 4)).astype(np.float32) / 2
    x = rng.normal(size=(3, 4, 3)).astype(np.float32)

    def f(xp, r):
        h = xp.tanh(xp.dot(r, W1))
        m = xp.add(xp.dot(h, W2), np.eye(4, dtype=np.float32) * 2)    # (4, 4), well conditioned
        return xp.add(xp.slogdet(m)[1], xp.sum(xp.square(h)))

    op = folx_amd.ParallelLaplacianOperator() if parallel else folx_amd.LoopLaplacianOperator()
    diag, grad = folx_amd.vmap(op(lambda r: f(fnp, r)))(x)
    assert diag.shape == (3, 12) and grad.shape == (3, 12)
    lap, jac = folx_amd.vmap(folx_amd.ForwardLaplacianOperator(0)(lambda r: f(fnp, r)))(x)
    np.testing.assert_allclose(diag.sum(1).numpy(), lap.numpy(), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(grad.numpy(), jac.numpy(), rtol=2e-4, atol=2e-5)
    for b in range(3):
        xb = torch.as_tensor(x[b], dtype=torch.float64).reshape(-1)
        fb = lambda z: f(plain, z.reshape(4, 3))
        H = torch.func.jacfwd(torch.func.jacrev(fb))(xb)
        np.testing.assert_allclose(diag[b].numpy(), torch.diagonal(H).numpy(), rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(grad[b].numpy(), torch.func.jacrev(fb)(xb).numpy(), rtol=2e-4, atol=2e-5)
    one_d, one_g = op(lambda r: f(fnp, r))(x[0])
    np.testing.assert_allclose(one_d.numpy(), diag[0].numpy(), rtol=1e-6)
    assert one_g.shape == (12,)


def test_value_only_functions():
    """argmax / argmin, logical functions, is_finite, trunc and integer conversion give plain
    values without derivatives (``warp_without_fwd_laplacian``,
    folx/wrapped_functions.py:445-449, :546-550)."""
    from folx_amd.api import BatchedArray

    x = np.random.default_rng(15).normal(size=(3, 4, 5)).astype(np.float32)
    seen = {}

    def f(r):
        h = fnp.sin(fnp.multiply(r, 2.0))
        seen['argmax'] = fnp.argmax(h, axis=-1)
        seen['argmin'] = fnp.argmin(h, axis=0)
        seen['finite'] = fnp.isfinite(h)
        seen['and'] = fnp.logical_and(fnp.greater(h, 0.0), fnp.less(h, 0.5))
        seen['not'] = fnp.logical_not(fnp.greater(h, 0.0))
        seen['int'] = fnp.astype(fnp.multiply(h, 3.0), np.int32)
        return fnp.sum(h)

    folx_amd.vmap(folx_amd.forward_laplacian(f, 0))(x)
    h = np.sin(2.0 * x)
    for v in seen.values():
        assert isinstance(v, BatchedArray)
    np.testing.assert_array_equal(seen['argmax'].data.numpy(), h.argmax(-1))
    np.testing.assert_array_equal(seen['argmin'].data.numpy(), h.argmin(1))
    assert seen['finite'].data.numpy().all()
    np.testing.assert_array_equal(seen['and'].data.numpy() != 0, (h > 0) & (h < 0.5))
    np.testing.assert_array_equal(seen['not'].data.numpy() != 0, ~(h > 0))
    np.testing.assert_array_equal(seen['int'].data.numpy(), np.trunc(3.0 * h))


def test_dense_times_sparse_keeps_the_sparse_rows(monkeypatch):
    """``mul`` of a dense-Jacobian triplet with a sparse one of the same shape goes to the
    kernel that reads the sparse rows in place; the result equals the densified rule."""
    from folx_amd import kernels as K

    calls = []
    orig = K.mul_sparse
    monkeypatch.setattr(K, 'mul_sparse', lambda *a: (calls.append(tuple(a[6].shape)), orig(*a))[1])
    rng = np.random.default_rng(16)
    W = rng.normal(size=(3, 4)).astype(np.float32)
    x = rng.normal(size=(2, 5, 3)).astype(np.float32)

    def fn(xp, r):
        env = xp.exp(xp.multiply(xp.dot(r, W), -0.3))                   # (5, 4), k = 3 per node
        mixed = xp.tanh(xp.add(env, xp.mean(env, axis=0, keepdims=True)))   # dense: every node sees all
        return xp.sum(xp.multiply(mixed, env))

    check_against_oracle(fn, x, 6)
    assert calls == [(3, 20)]


def test_slogdet_with_factor(monkeypatch):
    """``slogdet(A, factor=F)`` equals ``slogdet(A * F)``; with a dense A and a sparse F the product
    is left to the slogdet kernel, otherwise the mul rule runs first."""
    from folx_amd import kernels as K

    calls = []
    orig = K.slogdet
    monkeypatch.setattr(K, 'slogdet', lambda *a: (calls.append(len(a) > 4 and a[4] is not None), orig(*a))[1])
    rng = np.random.default_rng(17)
    W = rng.normal(size=(3, 4)).astype(np.float32)
    x = rng.normal(size=(2, 4, 3)).astype(np.float32)

    def fn(xp, r, dense_factor):
        env = xp.exp(xp.multiply(xp.dot(r, W), -0.3))                       # (4, 4), k = 3 per row
        h = xp.tanh(xp.add(env, xp.mean(env, axis=0, keepdims=True)))      # dense Jacobian
        A = xp.add(h, np.eye(4, dtype=np.float32) * 2)
        f = xp.add(env, xp.mean(env, axis=0, keepdims=True)) if dense_factor else env
        return xp.slogdet(A, factor=f)[1]

    check_against_oracle(lambda xp, r: fn(xp, r, False), x, 6)
    assert calls == [True]
    calls.clear()
    check_against_oracle(lambda xp, r: fn(xp, r, True), x, 6)       # the factor depends on every node: dense, mul rule first
    check_against_oracle(lambda xp, r: fn(xp, r, False), x, 0)      # everything dense
    assert True not in calls


def test_stagecheck_runs_every_kernel_call_against_its_fp64_rule():
    """tests/stagecheck.py on the stand-ins: every call is compared with the float64 rule of the
    same inputs, and a corrupted kernel is caught at its stage."""
    import folx_amd.kernels as K
    from stagecheck import StageCheck

    p = wl.psiformer_params(SMALL_PSI)
    x = wl.sample_electrons(2, SMALL_PSI.n_elec, 1.0, seed=3)
    fn = lambda xp, t: wl.psiformer_forward(p, t, xp)
    with StageCheck() as sc:
        run_product(fn, x, 6)
    used = sc.summary()
    assert {'dense', 'mhsa', 'slogdet'} <= set(used) or {'dense', 'mhsa_sparse', 'slogdet'} <= set(used), used
    assert all(w <= 1.0 for _, w, _ in used.values())
    good = K.elementwise
    K.elementwise = lambda *a, **k: tuple(t * (1 + 3e-5) for t in good(*a, **k))  # a 3e-5 relative error
    try:
        with pytest.raises(AssertionError, match='elementwise'):
            with StageCheck():
                run_product(lambda xp, t: xp.sum(xp.tanh(t)), x, 0)
    finally:
        K.elementwise = good


@pytest.mark.parametrize('thr', [0, 6])
def test_forward_laplacian_of_several_arguments(thr):
    """Two differentiated array arguments share one index space, numbered in argument order
    (folx/interpreter.py:319-340): the result equals the one-argument function of their
    concatenation; batched_vmap chunks both along the walker axis."""
    rng = np.random.default_rng(21)
    A, C = rng.normal(size=(3, 5)).astype(np.float32), rng.normal(size=(2, 5)).astype(np.float32)
    x, y = rng.normal(size=(5, 4, 3)).astype(np.float32), rng.normal(size=(5, 4, 2)).astype(np.float32)

    def two(xp, u, v):
        return xp.sum(xp.multiply(xp.tanh(xp.dot(u, A)), xp.sin(xp.dot(v, C))))

    def one(xp, z):  # z (4, 5) = [u | v] along the last axis, flattened argument by argument
        u = xp.reshape(xp.getitem(z, (slice(0, 12),)), (4, 3))
        v = xp.reshape(xp.getitem(z, (slice(12, 20),)), (4, 2))
        return two(xp, u, v)

    fl = folx_amd.forward_laplacian(lambda u, v: two(fnp, u, v), thr)
    got = folx_amd.vmap(fl)(x, y)
    z = np.concatenate([x.reshape(5, -1), y.reshape(5, -1)], axis=1)
    ref = one(ob, ob.init_state(z, dtype=np.float64))
    J = got.jacobian.dense_array.numpy()
    assert J.shape == (20, 5)
    np.testing.assert_allclose(got.x.numpy(), ref.x, rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(J, ref.J, rtol=1e-4, atol=1e-5)
    np.testing.assert_allclose(got.laplacian.numpy(), ref.lap, rtol=1e-4, atol=1e-5)
    chunked = folx_amd.batched_vmap(fl, 2)(x, y)
    np.testing.assert_allclose(chunked.laplacian.numpy(), got.laplacian.numpy(), rtol=1e-6)
    np.testing.assert_allclose(chunked.jacobian.dense_array.numpy(), J, rtol=1e-6, atol=1e-7)


def test_attention_beyond_the_kernel_sizes_runs_through_matmul_and_softmax():
    """n > 64 or d > 64 (or d % 4 != 0): the attention rule evaluates the same function from the
    two-operand product and softmax rules, masks included."""
    rng = np.random.default_rng(22)
    n, H, d = 5, 2, 6   # d % 4 != 0
    Wq, Wk, Wv = (rng.normal(size=(3, H * d)).astype(np.float32) / 2 for _ in range(3))
    x = rng.normal(size=(2, n, 3)).astype(np.float32)

    def fn(xp, t):
        q, k, v = (xp.reshape(xp.dot(t, w), (n, H, d)) for w in (Wq, Wk, Wv))
        return xp.sum(xp.tanh(xp.multi_head_self_attention(q, k, v)))

    check_against_oracle(fn, x, 0)
    check_against_oracle(fn, x, 6)
    masked_attention_beyond_kernel_sizes(run_product, lambda o: triplet_np(o))
    # the smallest shape of test/experimental/pallas/test_attention.py:323: one electron, one head of one feature
    masked_attention_beyond_kernel_sizes(run_product, lambda o: triplet_np(o), n=1, H=1, d=1, valid=1, B=1)


def masked_attention_beyond_kernel_sizes(run, to_np, n=5, H=2, d=6, valid=3, B=2):
    """A padded sequence (``valid`` of n electrons, the coordinates of the others inactive) at a shape the
    attention kernels do not take: scores of padding replaced by -1e20 in front of the softmax, Jacobian rows
    of inactive coordinates dropped (test/experimental/pallas/test_attention.py:320-326, reference_mhsa_kernel
    folx/experimental/pallas/attention/mhsa.py:79-94).  Rows of padding queries carry no meaning and are left
    out of the comparison, as in the reference's test."""
    rng = np.random.default_rng(24)
    Wq, Wk, Wv = (rng.normal(size=(3, H * d)).astype(np.float32) / 2 for _ in range(3))
    x = rng.normal(size=(B, n, 3)).astype(np.float32)
    mask = np.zeros((B, n), dtype=bool)
    mask[:, :valid] = True
    imask = np.zeros((3 * n, B), dtype=bool)
    imask[: 3 * valid] = True

    def fn(xp, t, m, im):
        q, k, v = (xp.reshape(xp.dot(t, w), (n, H, d)) for w in (Wq, Wk, Wv))
        return xp.multi_head_self_attention(xp.multiply(q, 1.0 / np.sqrt(d)), k, v, mask=m, input_mask=im)

    for thr in (0, 6):
        got = to_np(run(lambda xp, t: fn(xp, t, mask, imask), x, thr))
        ref = fn(ob, ob.init_state(x, dtype=np.float64), mask, imask)
        np.testing.assert_allclose(got[0][:, :valid], ref.x[:, :valid], rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(got[1][:, :, :valid], ref.J[:, :, :valid], rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(got[2][:, :valid], ref.lap[:, :valid], rtol=2e-4, atol=2e-4)
        assert np.isfinite(got[0]).all() and np.isfinite(got[1]).all() and np.isfinite(got[2]).all()
        assert not np.abs(got[1][3 * valid:]).any()   # rows of inactive coordinates


@pytest.mark.parametrize('name', sorted(BIG_MATRIX_FNS))
def test_matrix_rules_beyond_the_small_matrix_kernels(name):
    """slogdet / det / inv / solve of 34 x 34 matrices (the one-matrix-per-wavefront kernels stop at 32): the
    rules dispatch to their any-size forms (folx/slogdet.py:296-344, folx/linear_solve.py:54-145 take any n)."""
    x = (np.random.default_rng(23).normal(size=(2, 6)) * 0.3).astype(np.float32)
    check_against_oracle(BIG_MATRIX_FNS[name], x, 0)


@pytest.mark.parametrize('thr', [0, 6])
def test_generic_rule_built_from_a_torch_function(thr):
    """folx/wrapper.py:73-138, folx/wrapped_functions.py:597-618: a function without a rule of
    its own gets J_f J and J_f lap + sum_p J_p^T H_f J_p from autodiff (two arguments with
    Jacobians, a constant, a tuple of results); checked against the Hessian trace of the whole
    composition."""
    rng = np.random.default_rng(44)
    x = rng.normal(size=(3, 4, 3)).astype(np.float32)
    w = rng.normal(size=(3, 2)).astype(np.float32)

    def op(a, b, wc):  # per walker: a (4, 3), b (4,), wc (3, 2)
        z = torch.sin(a @ wc) * b[:, None]
        return z, torch.exp(-b) * a.sum()

    rule = folx_amd.wrap_forward_laplacian(op)
    folx_amd.register_function('my_op', rule)
    try:
        def model(r):
            h = fnp.tanh(r)
            s = fnp.sum(fnp.square(r), axis=-1)
            z, e = fnp.call('my_op', h, s, w)
            return fnp.add(fnp.sum(fnp.square(z)), fnp.sum(e))

        out = folx_amd.vmap(folx_amd.forward_laplacian(model, thr))(x)
    finally:
        folx_amd.deregister_function('my_op')

    def whole(t):
        z, e = op(torch.tanh(t), (t * t).sum(-1), torch.as_tensor(w, dtype=t.dtype))
        return (z * z).sum() + e.sum()

    by, bJ, bL = brute_force(whole, x.astype(np.float64))
    got = triplet_np(out)
    np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[1], bJ.reshape(got[1].shape), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-4)

    # a callable without a registered rule is wrapped on the fly; a linear one skips the Hessian term
    lin = folx_amd.wrap_forward_laplacian(lambda a: 2.0 * a.flip(0), flags=folx_amd.FunctionFlags.LINEAR)
    out2 = folx_amd.vmap(folx_amd.forward_laplacian(
        lambda r: fnp.sum(fnp.multiply(fnp.call(torch.cos, fnp.sin(r)), lin((fnp.sin(r),), {}, thr))), thr))(x)
    by, bJ, bL = brute_force(lambda t: (torch.cos(torch.sin(t)) * 2.0 * torch.sin(t).flip(0)).sum(), x.astype(np.float64))
    got = triplet_np(out2)
    np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[1], bJ.reshape(got[1].shape), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize('thr', [0, 16])
def test_custom_jac_hessian_jac_hook(thr):
    """folx/wrapper.py:73-138 with ``custom_jac_hessian_jac`` (folx/api.py:434-441): the hook's result replaces
    the automatic tr(J^T H J).  (i) test/test_layers.py:501-529: an identity whose hook returns 10 gives
    Laplacian 10, value and Jacobian untouched.  (ii) hand-written second-order terms that ARE the Hessian
    trace -- elementwise (``in_axes=()``: one element and its Jacobian column per call), along the last axis
    (``in_axes=-1``: rows), and the division rule's own form with two arguments (folx/custom_hessian.py:35-59)
    -- give what autodiff gives."""
    rng = np.random.default_rng(45)
    x = rng.normal(size=(2, 16)).astype(np.float32)

    ten = folx_amd.wrap_forward_laplacian(
        lambda a: 1.0 * a, custom_jac_hessian_jac=lambda args, extra, merge, idx: tuple(torch.full_like(t, 10.0) for t in args.x))
    folx_amd.register_function('identity', ten)
    try:
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda r: fnp.call('identity', r), thr))(x)
    finally:
        folx_amd.deregister_function('identity')
    np.testing.assert_allclose(out.x.numpy(), x)
    np.testing.assert_allclose(out.jacobian.dense_array.numpy(), np.eye(16)[:, None, :].repeat(2, 1), atol=1e-7)
    np.testing.assert_allclose(out.laplacian.numpy(), 10.0)

    y = rng.normal(size=(3, 4, 5)).astype(np.float32)

    def cube_hook(args, extra, merge, idx):       # f = a^3 elementwise: f'' = 6 a, tr = 6 a sum_p J_p^2
        (a,), (J,) = args.x, args.jacobian
        assert a.shape == () and J.data.dim() == 1
        return 6.0 * a * (J.data * J.data).sum()

    def sumsq_hook(args, extra, merge, idx):      # f = sum_k a_k^2 over the last axis: H = 2 I
        (a,), (J,) = args.x, args.jacobian
        assert a.dim() == 1 and J.data.dim() == 2
        return 2.0 * (J.data * J.data).sum()

    def div_hook(args, extra, merge, idx):        # f = a / b (folx/custom_hessian.py:35-59)
        a, b = merge(args.x, extra)
        Ja, Jb = (j.data for j in args.jacobian)
        return -2.0 / b**2 * (Ja * Jb).sum() + 2.0 * a / b**3 * (Jb * Jb).sum()

    cases = [
        (folx_amd.wrap_forward_laplacian(lambda a: a**3, in_axes=(), custom_jac_hessian_jac=cube_hook),
         lambda r, rule: fnp.sum(rule((fnp.sin(r),), {}, thr)), lambda t: (torch.sin(t) ** 3).sum()),
        (folx_amd.wrap_forward_laplacian(lambda a: (a * a).sum(-1), in_axes=-1, custom_jac_hessian_jac=sumsq_hook),
         lambda r, rule: fnp.sum(fnp.tanh(rule((fnp.sin(r),), {}, thr))), lambda t: torch.tanh((torch.sin(t) ** 2).sum(-1)).sum()),
        (folx_amd.wrap_forward_laplacian(lambda a, b: a / b, in_axes=(), custom_jac_hessian_jac=div_hook),
         lambda r, rule: fnp.sum(rule((fnp.sin(r), fnp.add(fnp.square(r), 1.0)), {}, thr)),
         lambda t: (torch.sin(t) / (t * t + 1.0)).sum()),
    ]
    for rule, model, whole in cases:
        got = triplet_np(folx_amd.vmap(folx_amd.forward_laplacian(lambda r: model(r, rule), thr))(y))
        by, bJ, bL = brute_force(whole, y.astype(np.float64))
        np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(got[1], bJ.reshape(got[1].shape), rtol=2e-4, atol=2e-5)
        np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-4)


def test_rules_that_carry_no_derivatives_or_act_elementwise():
    """folx/wrapper.py:141-176."""
    from folx_amd.api import BatchedArray

    x = np.random.default_rng(45).normal(size=(2, 5)).astype(np.float32)
    seen = {}

    def f(r):
        h = fnp.sin(r)
        seen['count'] = folx_amd.warp_without_fwd_laplacian(lambda t, thr_: (t > thr_).sum())((h, 0.25), {}, 0)
        y = folx_amd.wrap_elementwise(lambda t: -3.0 * t)((h,), {}, 0)
        return fnp.sum(fnp.square(y))

    out = folx_amd.vmap(folx_amd.forward_laplacian(f, 0))(x)
    assert isinstance(seen['count'], BatchedArray)
    np.testing.assert_array_equal(seen['count'].data.numpy(), (np.sin(x) > 0.25).sum(-1))
    by, bJ, bL = brute_force(lambda t: (9.0 * torch.sin(t) ** 2).sum(), x.astype(np.float64))
    got = triplet_np(out)
    np.testing.assert_allclose(got[0], by, rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[1], bJ.reshape(got[1].shape), rtol=2e-4, atol=2e-5)
    np.testing.assert_allclose(got[2], bL, rtol=2e-4, atol=2e-4)


def test_custom_jvp_rule_is_used_for_both_orders(monkeypatch):
    """test/test_customjvp.py:10-28: the rule differs from the true derivative by a factor of 2; value from the
    function, Jacobian from the rule, Laplacian from the rule's own derivative.  Without triplets the object is
    the plain function, and a missing rule is an error."""
    cpu_kernels.install(monkeypatch)

    @folx_amd.custom_jvp
    def fn(x):
        return torch.sin(x)

    with pytest.raises(AttributeError, match='defjvp'):
        folx_amd.vmap(folx_amd.forward_laplacian(fn, 0))(np.zeros((2, 3), dtype=np.float32))

    @fn.defjvp
    def fn_jvp(primals, tangents):
        (x,), (t,) = primals, tangents
        return fn(x), 2 * t * torch.cos(x)

    x = np.random.default_rng(3).normal(size=(3, 10)).astype(np.float32)
    for thr in (0, 10):
        out = folx_amd.vmap(folx_amd.forward_laplacian(fn, thr))(x)
        np.testing.assert_allclose(out.x.numpy(), np.sin(x), rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(out.jacobian.dense_array.numpy(), 2 * np.cos(x)[None] * np.eye(10)[:, None, :],
                                   rtol=1e-6, atol=1e-7)
        np.testing.assert_allclose(out.laplacian.numpy(), -2 * np.sin(x), rtol=1e-5, atol=1e-6)
    assert torch.equal(fn(torch.tensor([0.5])), torch.sin(torch.tensor([0.5])))
    with pytest.raises(NotImplementedError, match='cannot be traced'):
        folx_amd.vmap(folx_amd.forward_laplacian_torch(fn, 0))(x)


def test_auto_batched_vmap_without_a_gpu_runs_the_batch_whole(monkeypatch):
    """folx/experimental/vmap.py:14-73: with nothing to measure (host arrays) the batch is not cut; a cap still is."""
    cpu_kernels.install(monkeypatch)
    from folx_amd.experimental import auto_batched_vmap

    fl = folx_amd.forward_laplacian(lambda t: fnp.sum(fnp.tanh(fnp.multiply(t, t))), 0)
    x = np.random.default_rng(4).normal(size=(40, 6)).astype(np.float32)
    auto = auto_batched_vmap(fl)
    whole = folx_amd.vmap(fl)(x)
    assert torch.equal(auto(x).laplacian, whole.laplacian) and list(auto.chosen.values()) == [40]
    capped = auto_batched_vmap(fl, max_batch_size=7)
    np.testing.assert_allclose(capped(x).laplacian.numpy(), whole.laplacian.numpy(), rtol=1e-6, atol=1e-6)
    assert list(capped.chosen.values()) == [7]


def test_ad_helpers_have_the_reference_shapes_and_values():
    """test/test_ad.py:12-37: jacfwd flattens the input on the last axis, jacrev the output on the first, hessian is
    forward over reverse; values against torch.autograd.functional."""
    from folx_amd.ad import hessian, jacfwd, jacrev

    f = lambda x: torch.sin(x * x.sum())    # noqa: E731
    x = torch.as_tensor(np.random.default_rng(5).normal(size=(3, 4)))
    full = torch.autograd.functional.jacobian(f, x)                      # (3, 4, 3, 4)
    assert jacfwd(f)(x).shape == (3, 4, 12) and jacrev(f)(x).shape == (12, 3, 4)
    np.testing.assert_allclose(jacfwd(f)(x), full.reshape(3, 4, 12), rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(jacrev(f)(x), full.reshape(12, 3, 4), rtol=1e-12, atol=1e-13)
    v = x.reshape(12)
    H = hessian(f)(v)
    assert H.shape == (12, 12, 12)
    want = torch.stack([torch.autograd.functional.hessian(lambda z, i=i: f(z)[i], v) for i in range(12)])
    np.testing.assert_allclose(H, want, rtol=1e-11, atol=1e-12)
    # two arguments: jacrev gives one array per argument, jacfwd concatenates their entries
    g = lambda a, b: torch.tanh(a) * b.sum()    # noqa: E731
    a, b = x[0], x[1, :2]
    ra, rb = jacrev(g)(a, b)
    assert ra.shape == (4, 4) and rb.shape == (4, 2)
    np.testing.assert_allclose(jacfwd(g)(a, b), torch.cat([ra, rb], dim=1), rtol=1e-12, atol=1e-13)


def test_python_operators_on_triplets(monkeypatch):
    """A model written with Python operators only (the reference gets these from tracing jnp code): numpy and torch
    constants on either side (numpy defers to the reflected methods instead of broadcasting over the tuple), powers,
    comparisons, ``.T`` / ``.swapaxes`` / ``.mean``; also on values that are still deferred."""
    cpu_kernels.install(monkeypatch)
    rng = np.random.default_rng(0)
    W = rng.normal(size=(4, 5)).astype(np.float32)
    V = rng.normal(size=(3, 3)).astype(np.float32)
    c = rng.normal(size=(5,)).astype(np.float32)
    Vt, ct = torch.as_tensor(V), torch.as_tensor(c)

    def f(x):           # x (3, 4)
        h = fnp.tanh(x @ W)
        g = (V @ h) ** 2 + abs(h) ** 1.5 - 2.0 ** (h * 0.3) + c * h - c / (2.0 + h ** 2) + (Vt @ h) * ct
        m = fnp.where(h > 0.1, g, -g.T.T)
        lazy = fnp.dot(h, W.T.copy())                                   # a deferred product: the same sugar
        return (m / (1.0 + h.mean(axis=-1, keepdims=True) ** 2)).swapaxes(0, 1).sum(axis=0) + (lazy ** 2).T.sum(axis=0)[:3]

    def t(x):
        Wd, Vd, cd = (torch.as_tensor(a, dtype=x.dtype) for a in (W, V, c))
        h = torch.tanh(x @ Wd)
        g = (Vd @ h) ** 2 + abs(h) ** 1.5 - 2.0 ** (h * 0.3) + cd * h - cd / (2.0 + h ** 2) + (Vd @ h) * cd
        m = torch.where(h > 0.1, g, -g)
        return (m / (1.0 + h.mean(-1, keepdim=True) ** 2)).swapaxes(0, 1).sum(0) + ((h @ Wd.T) ** 2).T.sum(0)[:3]

    x = rng.normal(size=(2, 3, 4)).astype(np.float32)
    y, J, L = brute_force(t, x.astype(np.float64))
    for thr in (0, 4, 12):
        out = folx_amd.vmap(folx_amd.forward_laplacian(f, thr))(x)
        np.testing.assert_allclose(out.x.numpy(), y, rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(out.jacobian.dense_array.numpy(), J.reshape(tuple(out.jacobian.dense_array.shape)), rtol=2e-5, atol=2e-5)
        np.testing.assert_allclose(out.laplacian.numpy(), L, rtol=1e-4, atol=1e-4)
    with pytest.raises(TypeError):
        np.add(c, folx_amd.vmap(folx_amd.forward_laplacian(lambda z: z, 0))(x))   # numpy functions do not take triplets


def test_numpy_style_constants_and_full_reductions(monkeypatch):
    """The names the reference's tests take from jnp / lax around a model: constants and dtypes (numpy's own),
    ``max`` / ``min`` over all or some axes (module attributes that do not shadow the builtins), ``rem``,
    ``convert_element_type``, ``allclose``."""
    cpu_kernels.install(monkeypatch)
    x = np.random.default_rng(0).normal(size=(2, 3, 4)).astype(np.float32)

    def f(xp, t):
        return xp.add(xp.add(xp.max(xp.sin(t)), xp.sum(xp.min(t, axis=-1, keepdims=True))),
                      xp.sum(xp.multiply(xp.remainder(t, 0.7), np.eye(3, 4, dtype=np.float32))))

    check_against_oracle(lambda xp, t: f(xp if xp is not fnp else fnp, t) if xp is fnp else
                         xp.add(xp.add(xp.amax(xp.amax(xp.sin(t), axis=-1), axis=-1), xp.sum(xp.amin(t, axis=-1))),
                                xp.sum(xp.multiply(xp.remainder(t, 0.7), np.eye(3, 4, dtype=np.float32)))), x, 0)
    assert fnp.rem is fnp.remainder and fnp.zeros((2, 3)).shape == (2, 3) and fnp.eye(3).dtype == np.float64
    assert fnp.float32 is np.float32 and fnp.full_like(np.zeros((2, 2)), 3.0).tolist() == [[3.0, 3.0], [3.0, 3.0]]
    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fnp.convert_element_type(fnp.tanh(t), fnp.float64), 0))(x)
    assert fnp.allclose(out, np.tanh(x), atol=1e-6) and not fnp.allclose(out, np.tanh(x) + 1e-3)
    with pytest.raises(AttributeError):
        fnp.no_such_function


def test_scan_and_fori_loop_run_as_python_loops(monkeypatch):
    """``jax.lax.scan`` over constants (what the reference supports, folx/interpreter.py:133-184) and over a triplet, and
    ``fori_loop``: a small recurrent cell against the oracle running the same loop."""
    cpu_kernels.install(monkeypatch)
    rng = np.random.default_rng(6)
    W, U = rng.normal(size=(5, 5)).astype(np.float32) / 2, rng.normal(size=(3, 5)).astype(np.float32) / 2
    drive = rng.normal(size=(4, 3)).astype(np.float32)            # scanned-over constants
    V = rng.normal(size=(4, 5)).astype(np.float32)
    x = rng.normal(size=(2, 4, 5)).astype(np.float32)              # per walker: 4 time steps of 5 features (scanned triplet)

    def model(xp, t, scan, fori):
        cell = lambda h, u: (lambda hn: (hn, xp.sum(xp.square(hn))))(xp.tanh(xp.add(xp.dot(h, W), np.asarray(u) @ U)))
        h, ys = scan(cell, xp.getitem(t, 0), drive)                                        # constants scanned
        h2, ys2 = scan(lambda c, row: (xp.add(xp.multiply(c, 0.5), xp.sin(row)), None), h, t, reverse=True)   # a triplet scanned
        h3 = fori(1, 4, lambda i, c: xp.add(c, xp.multiply(xp.tanh(c), V[i])), h2)
        return xp.add(xp.sum(h3), xp.sum(ys)), ys2

    def with_loops(xp, t):
        if xp is fnp:
            return model(fnp, t, fnp.scan, fnp.fori_loop)[0]

        def py_scan(f, init, xs, reverse=False):
            n = xs.shape[0]
            carry, ys = init, [None] * n
            for i in (range(n - 1, -1, -1) if reverse else range(n)):
                carry, ys[i] = f(carry, xs[i] if isinstance(xs, np.ndarray) else xp.getitem(xs, i))
            return carry, (None if ys[0] is None else xp.stack(ys, axis=0))

        def py_fori(lo, hi, body, init):
            for i in range(lo, hi):
                init = body(i, init)
            return init

        return model(xp, t, py_scan, py_fori)[0]

    for thr in (0, 5, 20):
        check_against_oracle(with_loops, x, thr)
    out, ys2 = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: model(fnp, t, fnp.scan, fnp.fori_loop), 0))(x)
    assert ys2 is None and tuple(out.shape) == ()

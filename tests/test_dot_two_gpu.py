"""Two-operand ``dot_general`` on the GPU (folx/wrapped_functions.py:205-309): the batched
product kernel against the float64 oracle rule, and models written with plain ``matmul`` /
``einsum`` / ``softmax`` (test/test_layers.py:141-206, test/test_composite.py:45-83) against the
oracle and brute-force AD."""

import numpy as np
import pytest
import torch

from bruteforce import brute_force, plain
from one_constant_cases import ONE_CONSTANT_FNS
from oracle import backend as ob
from oracle import rules
from tolerances import assert_lap, assert_triplet, assert_val

import folx_amd
from folx_amd import numpy as fnp

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.float32).cuda()


def rand(rng, *shape):
    return rng.normal(size=shape).astype(np.float32)


@pytest.mark.parametrize('NB0,NB1,I,J,Kc,P', [
    (1, 1, 1, 1, 1, 1), (3, 2, 5, 7, 3, 4), (2, 4, 32, 32, 64, 12), (2, 1, 70, 45, 20, 3),
    (1, 2, 16, 16, 128, 2), (2, 2, 33, 31, 100, 5), (4, 1, 8, 8, 16, 0),
])
def test_dot_two_kernel(NB0, NB1, I, J, Kc, P):
    from folx_amd import kernels as K

    print(f'case dot_two NB=({NB0},{NB1}) I={I} J={J} K={Kc} P={P}', flush=True)
    rng = np.random.default_rng(41)
    a, aj, al = rand(rng, NB0, NB1, I, Kc), rand(rng, P, NB0, NB1, I, Kc), rand(rng, NB0, NB1, I, Kc)
    b, bj, bl = rand(rng, NB0, NB1, Kc, J), rand(rng, P, NB0, NB1, Kc, J), rand(rng, NB0, NB1, Kc, J)
    f64 = lambda *t: [np.asarray(v, dtype=np.float64) for v in t]
    ref = rules.dot_two_rule(*f64(a, aj, al, b, bj, bl))
    got = K.dot_two(dev(a), dev(aj), dev(al), dev(b), dev(bj), dev(bl))
    assert_triplet(got, ref, 'dot_two contiguous')
    # the same operands stored as (walker, electron, head, feature) and b transposed: q k^T read in place
    if P > 0:
        qa = lambda t, lead: dev(np.moveaxis(t, lead + 1, lead + 2))            # (.., NB0, I, NB1, Kc)
        qb = lambda t, lead: dev(np.moveaxis(np.swapaxes(t, -1, -2), lead + 1, lead + 2))  # (.., NB0, J, NB1, Kc)
        va = lambda t, lead: t.transpose(lead + 1, lead + 2)
        vb = lambda t, lead: t.transpose(lead + 1, lead + 2).transpose(-1, -2)
        got = K.dot_two(va(qa(a, 0), 0), va(qa(aj, 1), 1), va(qa(al, 0), 0),
                        vb(qb(b, 0), 0), vb(qb(bj, 1), 1), vb(qb(bl, 0), 0))
        assert_triplet(got, ref, 'dot_two strided views')


@pytest.mark.parametrize('B,Bt,I,J,Kc,P', [
    (1, 1, 1, 1, 1, 1), (3, 4, 5, 7, 3, 4), (2, 4, 32, 64, 64, 12), (2, 1, 70, 45, 20, 3),
    (2, 2, 33, 31, 100, 5), (4, 3, 8, 8, 16, 0),
    # contracted axes longer than the kernel's tile depth: slices of the contracted axis, added
    (2, 2, 9, 11, 130, 3), (1, 2, 16, 20, 300, 2),
])
def test_dot_const_kernel(B, Bt, I, J, Kc, P):
    """Batched product with a constant that has a batch axis (per-head weights) vs the float64 rule;
    the constant is read once per batch element (walker stride 0)."""
    from folx_amd import kernels as K

    print(f'case dot_const B={B} Bt={Bt} I={I} J={J} K={Kc} P={P}', flush=True)
    rng = np.random.default_rng(43)
    a, aj, al = rand(rng, B, Bt, I, Kc), rand(rng, P, B, Bt, I, Kc), rand(rng, B, Bt, I, Kc)
    W = rand(rng, Bt, Kc, J)
    f64 = lambda *t: [np.asarray(v, dtype=np.float64) for v in t]
    ref = rules.dot_const_rule(*f64(a, aj, al, W))
    got = K.dot_const(dev(a), dev(aj), dev(al), dev(W))
    assert_triplet(got, ref, 'dot_const contiguous')
    if P > 0:  # head-interleaved operand (walker, position, head, feature) viewed as (walker, head, position, feature)
        q = lambda t, lead: dev(np.moveaxis(t, lead + 1, lead + 2)).transpose(lead + 1, lead + 2)
        got = K.dot_const(q(a, 0), q(aj, 1), q(al, 0), dev(W))
        assert_triplet(got, ref, 'dot_const strided views')


@pytest.mark.parametrize('name', sorted(ONE_CONSTANT_FNS))
@pytest.mark.parametrize('sparse', [False, True])
def test_one_constant_products_in_models(name, sparse):
    """One operand with derivatives against a constant of any rank on either side, any contracted and
    batch axes (folx/wrapped_functions.py:71-171; test/test_layers.py:119-139, real half): oracle and
    brute-force AD, dense (threshold 0) and sparse (threshold = number of inputs)."""
    fn = ONE_CONSTANT_FNS[name]
    x = (0.7 * np.random.default_rng(9).normal(size=(3, 4, 3))).astype(np.float32)
    thr = 12 if sparse else 0
    print(f'case one-constant {name} thr={thr}', flush=True)
    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    J = out.jacobian.dense_array
    assert tuple(out.x.shape) == tuple(ref.x.shape)
    assert_val(out.x, ref.x, name + ' x')
    assert_val(J, ref.J[: J.shape[0]], name + ' jacobian')
    assert J.shape[0] == ref.J.shape[0] or np.abs(ref.J[J.shape[0]:]).max() == 0
    assert_lap(out.laplacian, ref.lap, name + ' laplacian')
    by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
    assert_val(out.x, by), assert_val(J, bJ[: J.shape[0]]), assert_lap(out.laplacian, bL)


def test_per_head_weights_at_model_size():
    """``einsum('nhd,hde->nhe')`` with per-head weights on a 32-electron, 4-head, 64-feature
    activation behind a dense layer, 96 dense Jacobian rows: one launch of the batched product
    with the constant operand, equal to the oracle."""
    from folx_amd import kernels as K

    rng = np.random.default_rng(12)
    W0 = rng.normal(size=(3, 256)).astype(np.float32) / 2
    Wh = rng.normal(size=(4, 64, 64)).astype(np.float32) / 8

    def fn(xp, x):
        h = xp.reshape(xp.tanh(xp.dot(x, W0)), (32, 4, 64))
        return xp.sum(xp.tanh(xp.einsum('nhd,hde->nhe', h, Wh)), axis=0)

    x = (0.7 * rng.normal(size=(2, 32, 3))).astype(np.float32)
    print('case per-head weights at model size', flush=True)
    with K.LaunchTimer() as lt:
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), 0))(x)
    assert 'dot_const_fwdlap' in {entry for (entry, _key) in lt.summary()}
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    assert_val(out.x, ref.x, 'per-head x')
    assert_val(out.jacobian.dense_array, ref.J, 'per-head jacobian')
    assert_lap(out.laplacian, ref.lap, 'per-head laplacian')


_ATT_W = [np.random.default_rng(40 + i).normal(size=(3, 8)).astype(np.float32) / 2 for i in range(3)]
_HEAD_W = [np.random.default_rng(50 + i).normal(size=(3, 4 * 32)).astype(np.float32) / 2 for i in range(3)]


def _heads(xp, x):
    """Multi-head attention written with plain einsum and softmax: 16 electrons, 4 heads of 32."""
    q, k, v = (xp.reshape(xp.dot(x, w), (16, 4, 32)) for w in _HEAD_W)
    s = xp.einsum('nhd,mhd->hnm', xp.multiply(q, 1.0 / np.sqrt(32.0)), k)
    o = xp.einsum('hnm,mhd->nhd', xp.softmax(s, axis=-1), v)
    return xp.sum(xp.tanh(xp.reshape(o, (16, 128))), axis=0)


MODELS = {
    # test/test_layers.py:141-171
    'attn': (lambda xp, x: xp.matmul(xp.exp(xp.matmul(xp.multiply(x, 0.3), xp.swapaxes(x, -2, -1))), x), (8, 3)),
    'rect': (lambda xp, x: xp.matmul(xp.sin(x), xp.cos(xp.swapaxes(x, -2, -1))), (8, 3)),
    # test/test_layers.py:173-206
    'ein_n1': (lambda xp, x: xp.einsum('nk,mk->nm', x, xp.sin(xp.getitem(x, (slice(0, 1),)))), (5, 3)),
    'ein_1n': (lambda xp, x: xp.einsum('nk,mk->nm', xp.getitem(x, (slice(0, 1),)), xp.sin(x)), (5, 3)),
    'ein_vec': (lambda xp, x: xp.einsum('k,mk->m', xp.getitem(x, (0,)), xp.sin(xp.getitem(x, (slice(0, 3),)))), (5, 3)),
    'ein_mpnn': (lambda xp, x: xp.einsum('ijh,jh->ih', xp.sin(xp.multiply(xp.expand_dims(x, 1), xp.expand_dims(x, 0))),
                                         xp.cos(x)), (5, 3)),
    # test/test_layers.py:119-139 with both operands depending on x
    'vec_mat': (lambda xp, x: xp.matmul(xp.getitem(x, (0,)), xp.swapaxes(xp.cos(x), -1, -2)), (4, 3)),
    # test/test_composite.py:45-83
    'softmax_attn': (lambda xp, x: xp.sum(xp.matmul(
        xp.softmax(xp.matmul(xp.dot(x, _ATT_W[0]), xp.swapaxes(xp.dot(x, _ATT_W[1]), -1, -2)), axis=-1),
        xp.dot(x, _ATT_W[2]))), (16, 3)),
    'heads': (_heads, (16, 3)),
}


@pytest.mark.parametrize('name', sorted(MODELS))
@pytest.mark.parametrize('sparse', [False, True])
def test_two_operand_products_in_models(name, sparse):
    """Dense (threshold 0) and sparse (threshold = number of inputs, as in the reference's tests)."""
    fn, shape = MODELS[name]
    x = (0.7 * np.random.default_rng(9).normal(size=(3, *shape))).astype(np.float32)
    thr = int(np.prod(shape)) if sparse else 0
    print(f'case two-operand {name} thr={thr}', flush=True)
    from folx_amd import kernels as K

    with K.LaunchTimer() as lt:
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
    used = {entry for (entry, _key) in lt.summary()}
    if not sparse:
        assert 'dot_two_fwdlap' in used, used   # dense Jacobians: the product is one rule, no (i, j, k) intermediate
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    J = out.jacobian.dense_array
    assert_val(out.x, ref.x, name + ' x')
    assert_val(J, ref.J[: J.shape[0]], name + ' jacobian')
    assert J.shape[0] == ref.J.shape[0] or np.abs(ref.J[J.shape[0]:]).max() == 0
    assert_lap(out.laplacian, ref.lap, name + ' laplacian')
    if name != 'heads':  # brute force over 48 inputs x 128 outputs is the oracle's job above
        by, bJ, bL = brute_force(lambda t: fn(plain, t), x.astype(np.float64))
        assert_val(out.x, by), assert_val(J, bJ[: J.shape[0]]), assert_lap(out.laplacian, bL)


def test_dot_two_at_attention_size_equals_multiply_and_sum():
    """Scores q k^T of the headline workload's shape (32 electrons, 4 heads of 64, 96 Jacobian
    rows) for 8 walkers: the product kernel and the multiply-and-sum decomposition through the
    mul and reduce_sum rules agree to rounding."""
    from folx_amd import wrapped_functions as wf
    from folx_amd.api import FwdJacobian, FwdLaplArray

    g = torch.Generator(device='cuda').manual_seed(3)
    B, H, n, d, P = 8, 4, 32, 64, 96
    rn = lambda *s: torch.randn(*s, device='cuda', generator=g)
    q = FwdLaplArray(rn(B, H, n, d), FwdJacobian(rn(P, B, H, n, d), None), rn(B, H, n, d))
    kt = FwdLaplArray(rn(B, H, d, n), FwdJacobian(rn(P, B, H, d, n), None), rn(B, H, d, n))
    print('case dot_two attention size', flush=True)
    with fnp.sparsity_threshold(0):
        got = wf._dot_two_operands(q, kt, 0)
        ref = wf._dot_mul_sum(q, kt, False, False)
    assert got.shape == (H, n, n)
    torch.testing.assert_close(got.x, ref.x, rtol=2e-5, atol=2e-5)
    torch.testing.assert_close(got.jacobian.data, ref.jacobian.data, rtol=2e-5, atol=1e-4)
    torch.testing.assert_close(got.laplacian, ref.laplacian, rtol=1e-4, atol=2e-2)

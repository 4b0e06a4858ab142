"""Sizes beyond what the specialised kernels are built for, on the GPU: matrices larger than 32 x 32 in slogdet /
det / inv / solve (composed from an any-size inverse and the batched product kernels; the reference takes any size,
folx/slogdet.py:296-344, folx/linear_solve.py:54-145) and masked attention on more than 64 positions (through the
product and softmax rules, folx/experimental/pallas/attention/mhsa.py:79-94 for the masks)."""

import numpy as np
import pytest
import torch

from oracle import backend as ob
from oracle import rules
from size_limit_cases import BIG_MATRIX_FNS
from tolerances import assert_lap, assert_triplet, assert_val

import folx_amd
from folx_amd import numpy as fnp

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=torch.float32).cuda()


def _matrices(rng, lead, n, P):
    A = (np.eye(n) * 2.0 + rng.normal(size=(*lead, n, n)) / np.sqrt(n)).astype(np.float32)
    if n >= 2:
        A[..., [0, 1], :] = A[..., [1, 0], :]     # a row exchange: the pivot search has work to do and the sign flips
    J = rng.normal(size=(P, *lead, n, n)).astype(np.float32)
    L = rng.normal(size=(*lead, n, n)).astype(np.float32)
    return A, J, L


@pytest.mark.parametrize('n,P,lead', [(33, 5, (3,)), (48, 7, (2, 2)), (64, 12, (4,)), (100, 3, (2,)),
                                      (120, 2, (1,)),      # beyond the LDS-resident size: elimination in global memory
                                      (130, 2, (2,)),      # contracted axis longer than one tile of the product kernel
                                      (5, 3, (2,)), (1, 2, (3,))])
def test_inv_values_and_composed_rules(n, P, lead):
    from folx_amd import kernels as K

    print(f'case any-size matrix rules n={n} P={P} lead={lead}', flush=True)
    rng = np.random.default_rng(100 + n)
    A, J, L = _matrices(rng, lead, n, P)
    f64 = lambda *t: [np.asarray(v, dtype=np.float64) for v in t]
    NM = int(np.prod(lead))
    Ainv, sign, ld = K.inv_values(dev(A).reshape(NM, n, n))
    s_ref, ld_ref = np.linalg.slogdet(A.astype(np.float64))
    assert_val(Ainv.reshape(*lead, n, n), np.linalg.inv(A.astype(np.float64)), 'inverse')
    np.testing.assert_array_equal(sign.cpu().numpy().reshape(lead), s_ref)
    assert_val(ld.reshape(lead), ld_ref, 'logdet')
    sref, ref = rules.slogdet_rule(*f64(A, J, L))
    gs, gld, gj, gl = K.slogdet_any(dev(A), dev(J), dev(L))
    np.testing.assert_array_equal(gs.cpu().numpy(), sref)
    # the allowance of test_slogdet: log|det| responds to rounding with the condition number
    cond = float(np.linalg.cond(A.astype(np.float64)).max())
    amp = max(1.0, cond / 50.0)
    from tolerances import LAP_ATOL, LAP_ATOL_REL, LAP_RTOL, VAL_ATOL_REL, VAL_RTOL

    def close(got, want, rtol, atol_rel, atol=0.0, what=''):
        want = np.asarray(want)
        np.testing.assert_allclose(got.cpu().numpy(), want, rtol=rtol * amp,
                                   atol=(atol + atol_rel * np.abs(want).max()) * amp, err_msg=what)

    close(gld, ref[0], VAL_RTOL, VAL_ATOL_REL, what='logdet')
    close(gj, ref[1], VAL_RTOL, VAL_ATOL_REL, what='logdet jacobian')
    close(gl, ref[2], LAP_RTOL, LAP_ATOL_REL, LAP_ATOL, what='logdet laplacian')
    iref = rules.inv_rule(*f64(A, J, L))
    gi = K.inv_any(dev(A), dev(J), dev(L))
    close(gi[0], iref[0], VAL_RTOL, VAL_ATOL_REL, what='inverse value')
    close(gi[1], iref[1], VAL_RTOL, VAL_ATOL_REL, what='inverse jacobian')
    close(gi[2], iref[2], LAP_RTOL, LAP_ATOL_REL, LAP_ATOL, what='inverse laplacian')
    if n <= K.SMALL_MATRIX_MAX:   # where both exist, the composed rule agrees with the one-matrix-per-wavefront kernel
        small = K.slogdet(dev(A), dev(J), dev(L))
        torch.testing.assert_close(gld, small[1], rtol=1e-5, atol=1e-5)
        torch.testing.assert_close(gj, small[2], rtol=1e-4, atol=1e-4)


def test_singular_and_permuted_matrices():
    """A permutation matrix scaled by 2 (sign = parity, log|det| = n log 2, inverse = transpose / 2) and a matrix with
    a zero row (sign 0, log|det| = -inf, as numpy.linalg.slogdet reports a singular matrix)."""
    from folx_amd import kernels as K

    n = 40
    perm = np.random.default_rng(3).permutation(n)
    A = np.zeros((2, n, n), dtype=np.float32)
    A[0, np.arange(n), perm] = 2.0
    A[1] = np.eye(n)
    A[1, 7] = 0.0
    Ainv, sign, ld = K.inv_values(dev(A))
    s_ref, ld_ref = np.linalg.slogdet(A.astype(np.float64))
    np.testing.assert_array_equal(sign.cpu().numpy(), s_ref)
    assert_val(ld[:1], ld_ref[:1], 'logdet of a scaled permutation')
    assert ld[1].item() == -np.inf
    np.testing.assert_allclose(Ainv[0].cpu().numpy(), A[0].T / 4.0, atol=1e-7)


@pytest.mark.parametrize('name', sorted(BIG_MATRIX_FNS))
def test_matrix_rules_in_models_beyond_32(name):
    fn = BIG_MATRIX_FNS[name]
    x = (np.random.default_rng(23).normal(size=(3, 6)) * 0.3).astype(np.float32)
    print(f'case 34 x 34 {name}', flush=True)
    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), 0))(x)
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    assert_val(out.x, ref.x, name + ' x')
    assert_val(out.jacobian.dense_array, ref.J, name + ' jacobian')
    assert_lap(out.laplacian, ref.lap, name + ' laplacian')


def test_attention_at_shapes_the_kernels_do_not_take():
    """d = 6 (no multiple of 4) with a padded sequence, and the smallest shape of
    test/experimental/pallas/test_attention.py:323 (one electron, one head of one feature)."""
    from test_host_logic import masked_attention_beyond_kernel_sizes

    run = lambda fn, x, thr: folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(torch.as_tensor(x).cuda())  # noqa: E731
    to_np = lambda o: (o.x.cpu().numpy().astype(np.float64), o.jacobian.dense_array.cpu().numpy().astype(np.float64),  # noqa: E731
                       o.laplacian.cpu().numpy().astype(np.float64))
    print('case attention n=5 H=2 d=6 valid=3', flush=True)
    masked_attention_beyond_kernel_sizes(run, to_np)
    print('case attention n=1 H=1 d=1', flush=True)
    masked_attention_beyond_kernel_sizes(run, to_np, n=1, H=1, d=1, valid=1, B=1)


def test_masked_attention_on_more_than_64_positions():
    """70 electrons of which 50 are real (the coordinates of the others inactive), 2 heads of 8: beyond the attention
    kernels' n <= 64, so the rule runs through the product and softmax rules with the masks applied; valid rows equal
    the oracle's (the padded-sequence case of test/experimental/pallas/test_attention.py:320-326 at a larger n)."""
    n, H, d, valid, B = 70, 2, 8, 50, 2
    rng = np.random.default_rng(24)
    Wq, Wk, Wv = (rng.normal(size=(3, H * d)).astype(np.float32) / 2 for _ in range(3))
    x = rng.normal(size=(B, n, 3)).astype(np.float32)
    mask = np.zeros((B, n), dtype=bool)
    mask[:, :valid] = True
    imask = np.zeros((3 * n, B), dtype=bool)
    imask[: 3 * valid] = True

    def fn(xp, t):
        q, k, v = (xp.reshape(xp.dot(t, w), (n, H, d)) for w in (Wq, Wk, Wv))
        return xp.multi_head_self_attention(xp.multiply(q, 1.0 / np.sqrt(d)), k, v, mask=mask, input_mask=imask)

    for thr in (0, 6):
        print(f'case masked attention n={n} thr={thr}', flush=True)
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(x)
        ref = fn(ob, ob.init_state(x, dtype=np.float64))
        J = out.jacobian.dense_array
        assert_val(out.x[:, :valid], ref.x[:, :valid], 'o')
        assert_val(J[:, :, :valid], ref.J[:, :, :valid], 'o_jac')
        assert_lap(out.laplacian[:, :valid], ref.lap[:, :valid], 'o_lap')
        assert torch.isfinite(out.x).all() and torch.isfinite(J).all() and torch.isfinite(out.laplacian).all()
        assert J[3 * valid:].abs().max().item() == 0.0

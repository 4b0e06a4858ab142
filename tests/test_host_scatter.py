"""Host logic of the scatter and min / max rules on CPU stand-ins for the kernels: every
case of the reference's test/test_scatter.py must agree with the dense oracle at sparsity
thresholds 0, 4 and 12, and keep a sparse Jacobian where the reference's test expects one
(test/test_scatter.py:30-31: ``x0_idx is not None`` at threshold = x.size)."""

import numpy as np
import pytest

import cpu_kernels
from oracle import backend as ob

import folx_amd
from folx_amd import index_algebra as ia
from folx_amd import numpy as fnp
import composed_cases
from scatter_cases import CASES, MIXED, fancy_take, min_max_elementwise
from test_host_logic import check_against_oracle, run_product


@pytest.fixture(autouse=True)
def _cpu(monkeypatch):
    cpu_kernels.install(monkeypatch)
    from folx_amd import sparse_ops

    sparse_ops.clear_caches()


X = np.random.default_rng(60).normal(size=(2, 12)).astype(np.float32)


@pytest.mark.parametrize('name', sorted(CASES))
@pytest.mark.parametrize('thr', [0, 12])
def test_scatter_cases(name, thr):
    check_against_oracle(CASES[name], X, thr)
    if thr == 12:
        out = run_product(CASES[name], X, thr)
        assert out.jacobian.weak, 'scatter lost the sparse Jacobian'


@pytest.mark.parametrize('name', sorted(MIXED))
@pytest.mark.parametrize('thr', [0, 4, 12])
def test_scatter_mixed_sparsity(name, thr):
    check_against_oracle(MIXED[name], X, thr)


@pytest.mark.parametrize('name', sorted(composed_cases.CASES))
@pytest.mark.parametrize('thr', [0, 12])
def test_composed_rules(name, thr):
    check_against_oracle(composed_cases.CASES[name], X, thr)


@pytest.mark.parametrize('name', ['lax_pad_interior', 'lax_pad_varying_value', 'lax_pad_negative', 'lax_pad_negative_interior',
                                  'flip_pad'])
def test_pad_keeps_the_jacobian_sparse(name):
    """Padding is an indexing operation (folx/wrapped_functions.py:480-487; test/test_layers.py:668-682 asserts
    ``is_jacobian_weak``, :763-776 one stored row): every output element is one operand element or the padding value."""
    out = run_product(composed_cases.CASES[name], X, 12)
    assert out.jacobian.weak and out.jacobian.data.shape[0] == 1


@pytest.mark.parametrize('thr', [0, 12])
def test_min_max(thr):
    check_against_oracle(min_max_elementwise, X, thr)


@pytest.mark.parametrize('thr', [0, 12])
def test_integer_array_indexing(thr):
    check_against_oracle(fancy_take, X, thr)
    if thr == 12:
        assert run_product(fancy_take, X, thr).jacobian.weak


def test_out_of_bounds_update_is_dropped():
    # test_scatter.py:52-54: .at[[1, 100]].add(x[:2] * 3) == .at[[1]].add(x[:1] * 3)
    got = lambda xp, x: xp.scatter(xp.sin(x), np.array([1, 100]),
                                   xp.multiply(xp.getitem(x, (slice(0, 2),)), 3.0), 'add')
    want = lambda xp, x: xp.scatter(xp.sin(x), np.array([1]),
                                    xp.multiply(xp.getitem(x, (slice(0, 1),)), 3.0), 'add')
    for thr in (0, 12):
        a = run_product(got, X, thr)
        ref = want(ob, ob.init_state(X, dtype=np.float64))
        np.testing.assert_allclose(a.x.numpy(), ref.x, rtol=1e-5, atol=1e-6)
        J = a.jacobian.dense_array.numpy()
        np.testing.assert_allclose(J, ref.J[: J.shape[0]], rtol=1e-5, atol=1e-6)
        np.testing.assert_allclose(a.laplacian.numpy(), ref.lap, rtol=1e-5, atol=1e-6)


def test_scatter_keeps_k_small():
    """Issue-#28 pattern (test_scatter.py:139-156): distances scattered into rows of zeros
    keep 3 dependencies per entry."""
    out = run_product(CASES['rows_into_zeros'], X, 6)
    assert out.jacobian.weak and out.jacobian.data.shape[0] == 3
    want = 3 * np.arange(4)[None, None, :] + np.arange(3)[:, None, None]
    np.testing.assert_array_equal(out.jacobian.x0_idx, np.broadcast_to(want, (3, 2, 4)))


def test_index_positions_matches_numpy():
    shape = (4, 3, 5)
    A = np.arange(60).reshape(shape)
    for idx in [0, (1, 2), slice(1, 3), (slice(None), 1), (np.array([0, 2]),),
                (np.array([0, 3, 0]), np.array([1, 2, 1])), (slice(None), np.array([[0, 1], [2, 2]])),
                (Ellipsis, np.array([4, 0])), (None, 1), (np.array([-1, 0]), slice(0, 2), 3)]:
        np.testing.assert_array_equal(ia.index_positions(shape, idx), A[idx])
    np.testing.assert_array_equal(ia.index_positions((12,), (np.array([1, 100, -13, -12]),)), [1, -1, -1, 0])

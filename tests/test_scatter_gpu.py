"""GPU parity of the position-gather entry point and the min / max binary functions against
numpy on the same inputs (kernel level), and of the scatter / min / max rules against the
dense fp64 oracle on the cases of the reference's test/test_scatter.py (model level)."""

import numpy as np
import pytest
import torch

from oracle import backend as ob
from oracle import rules
import composed_cases
from scatter_cases import CASES, MIXED, fancy_take, min_max_elementwise
from tolerances import assert_lap, assert_triplet, assert_val

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype).cuda()


@pytest.mark.parametrize('RB,S_in,S_out,n_slots,S_inner', [(7, 12, 12, 1, 1), (300, 5, 9, 3, 1), (4, 6, 4, 2, 3),
                                                           (5000, 33, 70, 6, 1), (3, 1, 1, 1, 1), (64, 40, 17, 1, 8)])
def test_gather_cols(RB, S_in, S_out, n_slots, S_inner):
    from folx_amd import kernels as K

    print(f'case gather_cols RB={RB} S_in={S_in} S_out={S_out} slots={n_slots} inner={S_inner}', flush=True)
    rng = np.random.default_rng(70)
    data = rng.normal(size=(RB, S_in * S_inner)).astype(np.float32)
    table = rng.integers(-1, S_in, size=(S_out, n_slots)).astype(np.int32)
    d3 = data.astype(np.float64).reshape(RB, S_in, S_inner)
    want = np.zeros((RB, S_out, S_inner))
    for s in range(n_slots):
        ok = table[:, s] >= 0
        want[:, ok] += d3[:, table[ok, s]]
    got = K.gather_cols(dev(data), dev(table, torch.int32), S_inner)
    assert_val(got, want.reshape(RB, -1), 'gather_cols')


@pytest.mark.parametrize('op', ['min', 'max'])
@pytest.mark.parametrize('shape,P', [((3, 5, 8), 7), ((2, 13), 1), ((4, 100, 10), 40)])
def test_binary_min_max(op, shape, P):
    from folx_amd import kernels as K

    print(f'case binary {op} {shape} P={P}', flush=True)
    rng = np.random.default_rng(71)
    a, b = (rng.normal(size=shape).astype(np.float32) for _ in range(2))
    b.reshape(-1)[::7] = a.reshape(-1)[::7]  # exact ties: half of each operand
    aj, bj = (rng.normal(size=(P, *shape)).astype(np.float32) for _ in range(2))
    al, bl = (rng.normal(size=shape).astype(np.float32) for _ in range(2))
    f = lambda *t: [np.asarray(v, dtype=np.float64) for v in t]
    want = rules.minmax_rule(*f(a, aj, al, b, bj, bl), is_max=(op == 'max'))
    got = K.binary(op, dev(a), dev(aj), dev(al), dev(b), dev(bj), dev(bl))
    assert_triplet(got, want, op)


def _run(fn, x, thr):
    import folx_amd
    from folx_amd import numpy as fnp

    out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: fn(fnp, t), thr))(torch.as_tensor(x).cuda())
    ref = fn(ob, ob.init_state(x, dtype=np.float64))
    J = out.jacobian.dense_array
    assert_val(out.x, ref.x, 'x')
    assert_val(J, ref.J[: J.shape[0]], 'jacobian')
    assert not np.abs(ref.J[J.shape[0]:]).any()
    assert_lap(out.laplacian, ref.lap, 'laplacian')
    return out


@pytest.mark.parametrize('name', sorted(CASES))
@pytest.mark.parametrize('thr', [0, 12])
def test_scatter_models(name, thr):
    print(f'case scatter model {name} thr={thr}', flush=True)
    x = np.random.default_rng(72).normal(size=(5, 12)).astype(np.float32)
    out = _run(CASES[name], x, thr)
    if thr == 12:
        assert out.jacobian.weak


@pytest.mark.parametrize('name', sorted(MIXED))
@pytest.mark.parametrize('thr', [0, 4, 12])
def test_scatter_mixed_models(name, thr):
    print(f'case scatter mixed model {name} thr={thr}', flush=True)
    _run(MIXED[name], np.random.default_rng(73).normal(size=(5, 12)).astype(np.float32), thr)


@pytest.mark.parametrize('name', sorted(composed_cases.CASES))
@pytest.mark.parametrize('thr', [0, 12])
def test_composed_rule_models(name, thr):
    print(f'case composed model {name} thr={thr}', flush=True)
    _run(composed_cases.CASES[name], np.random.default_rng(77).normal(size=(5, 12)).astype(np.float32), thr)


@pytest.mark.parametrize('thr', [0, 12])
def test_min_max_model(thr):
    print(f'case min/max model thr={thr}', flush=True)
    _run(min_max_elementwise, np.random.default_rng(74).normal(size=(6, 12)).astype(np.float32), thr)


@pytest.mark.parametrize('thr', [0, 12])
def test_integer_array_indexing_model(thr):
    print(f'case fancy take thr={thr}', flush=True)
    _run(fancy_take, np.random.default_rng(76).normal(size=(6, 12)).astype(np.float32), thr)


def test_scatter_large_batch_properties():
    """At a large batch: scatter-add of a gathered slice is linear in the updates, and a
    'set' followed by reading the same positions returns the updates."""
    import folx_amd
    from folx_amd import numpy as fnp

    B, n = 4096, 48
    x = np.random.default_rng(75).normal(size=(B, n)).astype(np.float32)
    idx = np.arange(0, n, 3)

    def f(t):
        upd = fnp.tanh(fnp.getitem(t, (slice(0, idx.size),)))
        y = fnp.scatter(fnp.sin(t), idx, upd, 'set')
        return fnp.getitem(y, (slice(0, n, 3),)), upd

    got, upd = folx_amd.vmap(folx_amd.forward_laplacian(f, n))(torch.as_tensor(x).cuda())
    torch.testing.assert_close(got.x, upd.x, rtol=0, atol=0)
    torch.testing.assert_close(got.laplacian, upd.laplacian, rtol=0, atol=0)
    torch.testing.assert_close(got.jacobian.dense_array, upd.jacobian.dense_array, rtol=0, atol=0)

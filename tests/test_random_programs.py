"""Random compositions of the rules (``tests/random_programs.py``): the product on the CPU stand-ins against the
oracle at several sparsity thresholds, the oracle against torch AD, and (``-m gpu``) the HIP path against the oracle."""

import numpy as np
import pytest
import torch

import cpu_kernels
import random_programs as rp
from bruteforce import brute_force, plain
from oracle import backend as ob

import folx_amd
from folx_amd import numpy as fnp


def _inputs(seed, walkers=2):
    return np.random.default_rng(1000 + seed).normal(size=(walkers, rp.N_IN)).astype(np.float32)


def _compare(out, ref, what):
    gx, gl = out.x.cpu().numpy().astype(np.float64), out.laplacian.cpu().numpy().astype(np.float64)
    J = out.jacobian.dense_array.cpu().numpy().astype(np.float64)
    P = ref.J.shape[0]
    if J.shape[0] < P:  # trailing inputs nothing depends on
        J = np.concatenate([J, np.zeros((P - J.shape[0], *J.shape[1:]))], 0)
    floor = lambda r: 2e-5 * max(1.0, float(np.abs(r).max()))
    np.testing.assert_allclose(gx, ref.x, rtol=2e-4, atol=floor(ref.x), err_msg=what)
    np.testing.assert_allclose(J, ref.J, rtol=2e-4, atol=floor(ref.J), err_msg=what)
    np.testing.assert_allclose(gl, ref.lap, rtol=2e-4, atol=10 * floor(ref.lap), err_msg=what)


@pytest.mark.parametrize('block', range(8))
def test_product_host_logic_against_the_oracle(block, monkeypatch):
    """50 programs per block (blocks 0-3: 7 steps, 4-5: 14 steps, 6-7: 9 steps with the second family of step
    kinds), thresholds 0 (dense), 2, 3, 5 and 12; the caches
    are NOT cleared between programs, so entries of one program meet the lookups of the next."""
    cpu_kernels.install(monkeypatch)
    from folx_amd import sparse_ops

    sparse_ops.clear_caches()
    for seed in range(50 * block, 50 * block + 50):
        steps = rp.generate(seed, (7, 7, 7, 7, 14, 14, 9, 9)[block], more=block >= 6)
        x = _inputs(seed)
        ref = rp.run(steps, ob, ob.init_state(x, dtype=np.float64))
        for thr in (0, 2, 3, 5, 12):
            out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: rp.run(steps, fnp, t), thr))(x)
            _compare(out, ref, f'seed {seed} thr {thr}: {rp.describe(steps)}')


def test_oracle_against_autograd_on_random_programs():
    """The oracle backend's rules in these combinations against the Hessian trace by torch AD in float64."""
    for seed in range(80):
        steps = rp.generate(seed, 7 if seed < 40 else 9, more=seed >= 40)
        x = _inputs(seed).astype(np.float64)
        ref = rp.run(steps, ob, ob.init_state(x, dtype=np.float64))
        by, bJ, bL = brute_force(lambda t: rp.run(steps, plain, t), x)
        what = f'seed {seed}: {rp.describe(steps)}'
        np.testing.assert_allclose(ref.x, by, rtol=1e-9, atol=1e-10, err_msg=what)
        np.testing.assert_allclose(ref.J, bJ.reshape(ref.J.shape), rtol=1e-8, atol=1e-9, err_msg=what)
        np.testing.assert_allclose(ref.lap, bL, rtol=1e-7, atol=1e-8, err_msg=what)


@pytest.mark.gpu
@pytest.mark.parametrize('block', range(4))
def test_hip_path_against_the_oracle(block):
    """The same programs on the GPU (5 walkers): every kernel the composed rules reach, in sequences nobody wrote by
    hand.  Block 2 starts from 64 inputs: row extents that are multiples of 4 take the 128-bit forms of the kernels;
    block 3 draws from the second family of step kinds too."""
    n_in = 64 if block == 2 else rp.N_IN
    for seed in range(30 * block, 30 * block + 30):
        steps = rp.generate(seed, (7, 14, 7, 9)[block], n_in, more=block == 3)
        x = np.random.default_rng(1000 + seed).normal(size=(5, n_in)).astype(np.float32)
        ref = rp.run(steps, ob, ob.init_state(x, dtype=np.float64))
        for thr in (0, 3, 12, 64)[:4 if block == 2 else 3]:
            print(f'random program seed {seed} thr {thr}: {rp.describe(steps)}', flush=True)
            out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: rp.run(steps, fnp, t), thr))(torch.as_tensor(x).cuda())
            _compare(out, ref, f'seed {seed} thr {thr}: {rp.describe(steps)}')


@pytest.mark.gpu
def test_graph_replay_of_random_programs_equals_eager_bit_for_bit():
    """``folx_amd.jit``: the first call runs eagerly, the second is captured, later ones replay; every call returns the
    bits of the eager run on the same input (fresh inputs per call)."""
    for seed in range(36):
        steps = rp.generate(seed, 8, 64 if seed % 3 == 0 else rp.N_IN, more=seed >= 24)
        n_in = 64 if seed % 3 == 0 else rp.N_IN
        thr = (0, 3, 12)[seed % 3]
        print(f'graph replay, random program seed {seed} thr {thr}: {rp.describe(steps)}', flush=True)
        eager = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: rp.run(steps, fnp, t), thr))
        fast = folx_amd.jit(folx_amd.vmap(folx_amd.forward_laplacian(lambda t: rp.run(steps, fnp, t), thr)))
        for call in range(4):
            x = torch.as_tensor(np.random.default_rng(7000 + seed + call).normal(size=(4, n_in)).astype(np.float32)).cuda()
            a, b = eager(x), fast(x)
            torch.cuda.synchronize()
            assert torch.equal(a.x, b.x) and torch.equal(a.laplacian, b.laplacian), f'seed {seed} call {call}'
            assert torch.equal(a.jacobian.dense_array, b.jacobian.dense_array), f'seed {seed} call {call}'


def test_traced_front_door_on_random_programs(monkeypatch, caplog):
    """The same programs written with torch (``bruteforce.plain``), traced by ``forward_laplacian_torch`` and evaluated
    through the rules, against the oracle; no equation may fall back to the generic rule."""
    cpu_kernels.install(monkeypatch)
    with caplog.at_level('WARNING'):
        for seed in range(100):
            steps = rp.generate(seed, (8, 14, 9)[(seed >= 40) + (seed >= 60)], more=seed >= 60)
            x = _inputs(seed)
            ref = rp.run(steps, ob, ob.init_state(x, dtype=np.float64))
            for thr in (0, 3, 12):
                out = folx_amd.vmap(folx_amd.forward_laplacian_torch(lambda t: rp.run(steps, plain, t), thr))(x)
                _compare(out, ref, f'traced, seed {seed} thr {thr}: {rp.describe(steps)}')
    assert not [r for r in caplog.records if 'no forward-Laplacian rule' in r.message]


@pytest.mark.gpu
def test_traced_front_door_on_random_programs_on_the_gpu():
    for seed in range(45):
        steps = rp.generate(seed, 8, more=seed >= 30)
        x = _inputs(seed, walkers=5)
        ref = rp.run(steps, ob, ob.init_state(x, dtype=np.float64))
        for thr in (0, 12):
            print(f'traced random program seed {seed} thr {thr}: {rp.describe(steps)}', flush=True)
            out = folx_amd.vmap(folx_amd.forward_laplacian_torch(lambda t: rp.run(steps, plain, t), thr))(torch.as_tensor(x).cuda())
            _compare(out, ref, f'traced, seed {seed} thr {thr}: {rp.describe(steps)}')

"""Seeded random stacks of the fused layer rules at awkward widths: three Dense layers whose widths are drawn from
1 ... 130 (multiples of 16 and not, below and above the 128-column limit of the narrow kernels), each optionally behind a
LayerNorm, followed by an activation and a skip connection, then one of eight tails (reductions, softmax, logsumexp, a
sliced product, a concatenation, a maximum).  Checked against the float64 oracle; where a draw is ill-conditioned (a
LayerNorm over nearly equal entries) the bar is the float32 oracle's own distance from float64, times 8."""

import numpy as np
import pytest
import torch

import cpu_kernels
from oracle import backend as ob

import folx_amd
from folx_amd import numpy as fnp

WIDTHS = [1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 31, 32, 33, 48, 64, 65, 100, 128, 130]


def draw(seed):
    rng = np.random.default_rng(seed)
    n, f_in, B = int(rng.integers(1, 9)), int(rng.integers(1, 7)), int(rng.integers(1, 6))
    dims = [int(rng.choice(WIDTHS)) for _ in range(3)]
    Ws = [rng.normal(size=(a, b)).astype(np.float32) / np.sqrt(a) for a, b in zip([f_in] + dims[:-1], dims)]
    bs = [rng.normal(size=(b,)).astype(np.float32) * 0.1 if rng.random() < 0.7 else None for b in dims]
    acts = [str(rng.choice(['tanh', 'silu', 'none', 'sin', 'sigmoid'])) for _ in dims]
    use_ln = [bool(rng.random() < 0.4) for _ in dims]
    res = [bool(rng.random() < 0.4) for _ in dims]
    tail = str(rng.choice(['sum_all', 'sum_last', 'mean_first', 'softmax_sum', 'logsumexp', 'slice_dot', 'concat', 'max']))
    x = rng.normal(size=(B, n, f_in)).astype(np.float32)

    def f(xp, h):
        for i, (W, b, act) in enumerate(zip(Ws, bs, acts)):
            hin = xp.layer_norm(h, None, None, 1e-5) if use_ln[i] and h.shape[-1] > 3 else h
            z = xp.dot(hin, W, b) if b is not None else xp.dot(hin, W)
            if act != 'none':
                z = getattr(xp, act)(z)
            h = xp.add(z, h) if res[i] and z.shape == h.shape else z
        half = max(1, h.shape[-1] // 2)
        return {
            'sum_all': lambda: xp.sum(h), 'sum_last': lambda: xp.sum(h, axis=-1), 'mean_first': lambda: xp.mean(h, axis=0),
            'softmax_sum': lambda: xp.sum(xp.multiply(xp.softmax(h, axis=-1), h), axis=-1),
            'logsumexp': lambda: xp.logsumexp(h, axis=-1)[0],
            'slice_dot': lambda: xp.dot(xp.getitem(h, (slice(None), slice(0, half))), np.ones((half, 3), np.float32)),
            'concat': lambda: xp.sum(xp.concatenate([h, xp.tanh(h)], axis=-1), axis=0),
            'max': lambda: xp.amax(h, axis=-1),
        }[tail]()

    what = f'seed {seed}: n {n} f_in {f_in} B {B} widths {dims} {acts} LayerNorm {use_ln} skip {res} tail {tail}'
    return f, x, (0, f_in, n * f_in), what


def check(seed, device):
    f, x, thresholds, what = draw(seed)
    r64 = f(ob, ob.init_state(x, dtype=np.float64))
    r32 = f(ob, ob.init_state(x, dtype=np.float32))
    for thr in thresholds:
        out = folx_amd.vmap(folx_amd.forward_laplacian(lambda t: f(fnp, t), thr))(torch.as_tensor(x).to(device))
        J = out.jacobian.dense_array.cpu().numpy().astype(np.float64)
        if J.shape[0] < r64.J.shape[0]:
            J = np.concatenate([J, np.zeros((r64.J.shape[0] - J.shape[0], *J.shape[1:]))], 0)
        for name, got, ref, ref32, rtol in (('value', out.x.cpu().numpy(), r64.x, r32.x, 1e-5), ('jacobian', J, r64.J, r32.J, 1e-5),
                                            ('laplacian', out.laplacian.cpu().numpy(), r64.lap, r32.lap, 1e-4)):
            scale = max(1.0, float(np.abs(ref).max()))
            floor = max(2e-6 * scale * (10 if name == 'laplacian' else 1), 8 * float(np.abs(ref32 - ref).max()))
            np.testing.assert_allclose(got, ref, rtol=rtol, atol=floor, err_msg=f'{name}, thr {thr}, {what}')


@pytest.mark.parametrize('block', range(2))
def test_layer_stacks_host_logic(block, monkeypatch):
    cpu_kernels.install(monkeypatch)
    for seed in range(60 * block, 60 * block + 60):
        check(seed, 'cpu')


@pytest.mark.gpu
@pytest.mark.parametrize('block', range(4))
def test_layer_stacks_on_the_gpu(block):
    for seed in range(100 * block, 100 * block + 100):
        print(f'layer stack {draw(seed)[3]}', flush=True)
        check(seed, 'cuda')

"""GPU parity of every C-ABI entry point against the fp64 oracle on the same seeded fp32
inputs.  All calls go through libfolx_hip.so (folx_amd.kernels -> ctypes)."""

import numpy as np
import pytest
import torch

from oracle import index_algebra as ia
from oracle import rules
from tolerances import assert_lap, assert_triplet, assert_val

pytestmark = pytest.mark.gpu


def dev(a, dtype=torch.float32):
    return torch.as_tensor(np.ascontiguousarray(a), dtype=dtype).cuda()


def f64(*arrs):
    return [np.asarray(a, dtype=np.float64) for a in arrs]


def rand(rng, *shape):
    return rng.normal(size=shape).astype(np.float32)


POSITIVE = {'log', 'sqrt', 'rsqrt', 'log1p', 'reciprocal', 'cbrt'}
UNIT = {'asin', 'acos', 'atanh', 'erf_inv'}
ACTS = ['tanh', 'silu', 'exp', 'log', 'sqrt', 'rsqrt', 'square', 'logistic', 'softplus', 'sin', 'cos',
        'abs', 'log1p', 'reciprocal', 'expm1', 'sinh', 'cosh', 'tan', 'asin', 'acos', 'atan', 'asinh', 'acosh',
        'atanh', 'erf', 'erfc', 'erf_inv', 'cbrt', 'lgamma', 'digamma']


@pytest.mark.parametrize('name', ACTS)
@pytest.mark.parametrize('shape,P', [((3, 5, 8), 7), ((2, 13), 1), ((4, 100, 100), 40)])
def test_elementwise(name, shape, P):
    from folx_amd import kernels as K

    print(f'case elementwise {name} {shape} P={P}', flush=True)
    rng = np.random.default_rng(0)
    x, J, L = rand(rng, *shape), rand(rng, P, *shape), rand(rng, *shape)
    if name in POSITIVE:
        x = np.abs(x) + 0.2
    if name in UNIT:
        x = rng.uniform(-0.9, 0.9, size=shape).astype(np.float32)
    if name == 'acosh':
        x = np.abs(x) + 1.2
    if name in ('tan', 'sinh', 'cosh'):
        x = np.clip(x, -1.3, 1.3)   # stay away from the poles / large magnitudes of fp32
    if name in ('lgamma', 'digamma'):   # positive arguments, and negative ones away from the poles
        neg = (rng.integers(-3, 0, size=shape) + rng.uniform(0.25, 0.75, size=shape)).astype(np.float32)
        x = np.where(rng.uniform(size=shape) < 0.3, neg, rng.uniform(0.3, 9.0, size=shape).astype(np.float32))
    ref = rules.elementwise_rule(name, *f64(x, J, L))
    got = K.elementwise(name, dev(x), dev(J), dev(L))
    assert_triplet(got, ref, name)
    # in-place use is part of the contract
    tx, tJ, tL = dev(x), dev(J), dev(L)
    got2 = K.elementwise(name, tx, tJ, tL, inplace=True)
    assert got2[0].data_ptr() == tx.data_ptr()
    assert_triplet(got2, ref, name + ' in-place')


@pytest.mark.parametrize('c', [2.5, -0.5, 1.0 / 3.0])
def test_pow_constant_exponent(c):
    from folx_amd import kernels as K

    rng = np.random.default_rng(1)
    x, J, L = np.abs(rand(rng, 6, 9)) + 0.5, rand(rng, 5, 6, 9), rand(rng, 6, 9)
    ref = rules.elementwise_rule('pow', *f64(x, J, L), c)
    got = K.elementwise('pow', dev(x), dev(J), dev(L), param=c)
    assert_triplet(got, ref, f'pow {c}')


@pytest.mark.parametrize('n', [2, 3, -1, -2, 5])
def test_integer_pow(n):
    from folx_amd import kernels as K

    rng = np.random.default_rng(1)
    x, J, L = np.abs(rand(rng, 6, 9)) + 0.5, rand(rng, 5, 6, 9), rand(rng, 6, 9)
    ref = rules.elementwise_rule('integer_pow', *f64(x, J, L), n)
    got = K.elementwise('integer_pow', dev(x), dev(J), dev(L), param=n)
    assert_triplet(got, ref, f'integer_pow {n}')


DENSE_CASES = [
    # (rows shape, P, K, N, bias)
    ((20, 100), 8, 4, 100, True),      # first layer of the README MLP (K = 4)
    ((3, 100), 40, 100, 100, True),    # hidden layer (K = N = 100, not a tile multiple)
    ((3, 100), 12, 100, 1, False),     # output layer (N = 1)
    ((5, 32), 9, 256, 256, True),      # PsiFormer width
    ((2, 7), 3, 17, 33, True),         # odd sizes: scalar load paths
    ((1, 1), 1, 1, 1, False),
    ((2, 64), 6, 512, 512, False),     # large-config width
    ((4, 16), 5, 64, 48, True),        # BN = 64 variant
    # direct-to-LDS path (K % 16 == 0, N % 4 == 0) at its edges
    ((1, 3), 2, 16, 4, True),          # one chunk, narrowest output
    ((3, 50), 7, 48, 100, True),       # odd number of chunks, clamped column loads
    ((3, 50), 4, 832, 256, False),     # long K, ragged last row tile
    ((2, 70), 3, 32, 260, True),       # two column tiles, the second nearly empty
    ((1, 130), 5, 64, 20, False),      # BN = 32 variant, more rows than one tile
    # narrow outputs; N = 1 with K % 4 == 0 is a matrix-vector kernel without MFMA
    ((5, 33), 7, 64, 3, True),
    ((2, 70), 3, 256, 4, True),
    ((20, 100), 40, 100, 1, True),     # last layer of the README MLP
    ((1, 1), 0, 4, 2, False),
    ((1, 1), 0, 4, 1, False),          # one row, one 128-bit load
    ((3, 37), 5, 300, 1, True),        # K > 256: one row per 32 lanes, three passes over K
    ((3, 50), 2, 256, 1, False),       # widest K of the flat-run kernel, ragged last block of rows
    ((2, 9), 3, 18, 1, True),          # K % 4 != 0: N = 1 through the GEMM
]


@pytest.mark.parametrize('rows,P,Kd,N,bias', DENSE_CASES)
def test_dense(rows, P, Kd, N, bias):
    from folx_amd import kernels as K

    print(f'case dense rows={rows} P={P} K={Kd} N={N}', flush=True)
    rng = np.random.default_rng(2)
    x, J, L = rand(rng, *rows, Kd), rand(rng, P, *rows, Kd), rand(rng, *rows, Kd)
    W = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32)
    b = rand(rng, N) if bias else None
    ref = rules.dense_rule(*f64(x, J, L, W), None if b is None else b.astype(np.float64))
    got = K.dense(dev(x), dev(J), dev(L), dev(W), None if b is None else dev(b))
    assert_triplet(got, ref, 'dense')


def test_floor_is_used_by_small_entries_only():
    """The absolute floors of the parity bars (tests/tolerances.py) are meant for entries that cancel to near zero.
    On a width-256 layer: the entries of the GEMM's Jacobian output that need the floor are few and all small
    (below 5 % of the largest entry), and the kernel's error as a whole is that of a float32 product -- its rms
    distance from the float64 product is within 1.5 x that of numpy's float32 product of the same operands, so a
    kernel uniformly worse than float32 rounding cannot hide under the floor.  The same for the fused tanh rule."""
    from folx_amd import kernels as K
    from tolerances import VAL_RTOL, floor_usage

    rng = np.random.default_rng(21)
    rows, P, Kd, N = (4, 32), 96, 256, 256
    x, J, L = rand(rng, *rows, Kd), rand(rng, P, *rows, Kd), rand(rng, *rows, Kd)
    W = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32)
    ref = rules.dense_rule(*f64(x, J, L, W))
    got = K.dense(dev(x), dev(J), dev(L), dev(W))
    gJ = got[1].cpu().numpy().astype(np.float64)
    frac, small = floor_usage(gJ, ref[1], VAL_RTOL)
    rms = lambda a: float(np.sqrt(np.mean(np.square(a))))
    e_gpu, e_np = rms(gJ - ref[1]), rms((J @ W).astype(np.float64) - ref[1])
    print(f'dense K=256: {100 * frac:.2f} % of the Jacobian entries need the floor, all below {100 * small:.2f} % of the '
          f'largest entry; rms error {e_gpu:.2e} (numpy float32: {e_np:.2e})', flush=True)
    assert frac < 0.05 and small < 0.05
    assert e_gpu <= 1.5 * e_np
    got = K.elementwise('tanh', *[dev(t.astype(np.float32)) for t in ref])
    ref32 = rules.elementwise_rule('tanh', *[t.astype(np.float32) for t in ref])
    zf = rules.elementwise_rule('tanh', *[t.astype(np.float32).astype(np.float64) for t in ref])
    gJ = got[1].cpu().numpy().astype(np.float64)
    frac, small = floor_usage(gJ, zf[1], VAL_RTOL)
    e_gpu, e_np = rms(gJ - zf[1]), rms(ref32[1].astype(np.float64) - zf[1])
    print(f'tanh: {100 * frac:.2f} % need the floor (below {100 * small:.2f} % of the largest entry); rms error '
          f'{e_gpu:.2e} (numpy float32: {e_np:.2e})', flush=True)
    assert frac < 0.05 and small < 0.05
    assert e_gpu <= 2.0 * e_np


DENSE_ACT_CASES = [
    # (rows shape, P, K, N, bias, act)
    ((20, 100), 400, 100, 100, True, 'silu'),   # README MLP hidden layer: Jacobian rows split over workgroups
    ((20, 100), 400, 4, 100, True, 'silu'),     # its first layer (K = 4)
    ((7, 100), 4, 100, 100, True, 'silu'),      # sparse storage of the same layer (4 rows)
    ((3, 256), 6, 32, 32, True, 'tanh'),        # two-electron stream: 4 row strips, one column strip
    ((1, 130), 5, 64, 64, False, 'tanh'),       # two column strips, ragged last row tile
    ((2, 33), 9, 128, 128, True, 'softplus'),   # widest layer the kernel takes
    ((1, 50), 17, 96, 20, True, 'logistic'),    # K / 4 even but not a power of two
    ((1, 70), 3, 36, 33, True, 'exp'),          # K % 8 == 4, N just past one strip
    ((1, 1), 0, 8, 1, False, 'sin'),            # no Jacobian rows, one row, one column
    ((5, 40), 64, 16, 128, True, 'cos'),
    ((2, 64), 31, 104, 100, False, 'square'),   # odd number of Jacobian rows
    ((1, 64), 100, 100, 100, True, 'tanh'),     # one row tile, many groups
    # a short tail of columns behind full strips (the last strip is mostly padding), 16+ Jacobian rows
    ((1, 70), 40, 100, 98, True, 'silu'),       # tail of 2 columns, last tile of 6 rows
    ((3, 50), 17, 68, 33, True, 'tanh'),        # one strip + 1 column, K = 68
    ((1, 200), 16, 96, 68, False, 'softplus'),  # two strips + 4 columns
    ((1, 5), 20, 100, 97, True, 'exp'),         # fewer rows than a tile
    ((2, 48), 24, 100, 100, True, 'sin'),
    # wide layers (N > 128): tiles of 4 positions x 32 Jacobian rows, activation in the GEMM's epilogue
    ((2, 32), 96, 256, 256, True, 'tanh'),      # transformer MLP: three full groups of 32 Jacobian rows
    ((3, 16), 48, 832, 256, True, 'tanh'),      # one-electron stream: three groups of 16 Jacobian rows
    ((1, 8), 5, 16, 132, False, 'silu'),        # one chunk of K, column tile cut at 132, one partial group of 16
    ((1, 12), 33, 64, 512, True, 'softplus'),   # two column tiles, 1 row in the second group
    ((1, 4), 64, 48, 300, True, 'sin'),         # second column tile cut at 44 columns
    ((5, 4), 1, 32, 256, False, 'square'),      # a single Jacobian row
    ((2, 8), 40, 64, 300, True, 'tanh'),        # groups of 16 Jacobian rows, the last one half full, cut column tile
    ((4, 16), 16, 48, 256, True, 'logistic'),   # exactly one group of 16
]


@pytest.mark.parametrize('rows,P,Kd,N,bias,act', DENSE_ACT_CASES)
def test_dense_act(rows, P, Kd, N, bias, act):
    """Dense layer + activation as one kernel against the composition of the two oracle rules."""
    from folx_amd import kernels as K

    print(f'case dense_act rows={rows} P={P} K={Kd} N={N} act={act}', flush=True)
    rng = np.random.default_rng(21)
    x, J, L = rand(rng, *rows, Kd), rand(rng, P, *rows, Kd), rand(rng, *rows, Kd)
    W = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32)
    b = rand(rng, N) if bias else None
    z = rules.dense_rule(*f64(x, J, L, W), None if b is None else b.astype(np.float64))
    ref = rules.elementwise_rule(act, *z)
    assert K.dense_act_supported(act, Kd, N, rows=int(np.prod(rows)))
    for rep in range(2):  # the second call finds the counters as the first one left them
        got = K.dense_act(act, dev(x), dev(J), dev(L), dev(W), None if b is None else dev(b))
        assert_triplet(got, ref, f'dense_act call {rep}')
    if K.dense_act_residual_supported(Kd, N):  # narrow layers add a skip connection in their epilogue
        res = (rand(rng, *rows, N), rand(rng, P, *rows, N), rand(rng, *rows, N))
        got = K.dense_act(act, dev(x), dev(J), dev(L), dev(W), None if b is None else dev(b), 0.0,
                          tuple(dev(t) for t in res))
        assert_triplet(got, tuple(a + r.astype(np.float64) for a, r in zip(ref, res)), 'dense_act + residual')


def test_dense_act_matches_two_kernels_large():
    """At a full-size batch the fused kernel and dense + elementwise agree to rounding."""
    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(5)
    R, P, Kd, N = 256 * 100, 4, 100, 100
    x = torch.randn(R, Kd, device='cuda', generator=g)
    J = torch.randn(P, R, Kd, device='cuda', generator=g)
    L = torch.randn(R, Kd, device='cuda', generator=g)
    W = torch.randn(Kd, N, device='cuda', generator=g) / 10
    b = torch.randn(N, device='cuda', generator=g)
    got = K.dense_act('silu', x, J, L, W, b)
    ref = K.elementwise('silu', *K.dense(x, J, L, W, b))
    for a, r, nm in zip(got, ref, ('x', 'jac', 'lap')):
        torch.testing.assert_close(a, r, rtol=2e-5, atol=2e-5, msg=lambda m: f'{nm}: {m}')


NORM_DENSE_CASES = [
    # (rows shape, P, K, N, gamma/beta, bias, act)
    ((2, 32), 96, 256, 256, True, False, None),      # transformer q / k / v projection behind LayerNorm
    ((2, 32), 96, 256, 256, True, True, 'tanh'),     # transformer MLP behind LayerNorm
    ((1, 8), 40, 64, 132, False, True, None),        # no gamma / beta, partial group of Jacobian rows, cut column tile
    ((1, 12), 33, 512, 512, True, True, 'silu'),     # widest K, two column tiles, 1 row in the second group
    ((3, 4), 1, 16, 300, True, False, 'softplus'),   # one chunk of K, one Jacobian row
    ((1, 4), 64, 48, 256, True, True, 'sin'),
]


@pytest.mark.parametrize('rows,P,Kd,N,affine,bias,act', NORM_DENSE_CASES)
def test_norm_dense(rows, P, Kd, N, affine, bias, act):
    """LayerNorm + dense (+ activation) as one rule against the chain of oracle rules."""
    from oracle import backend as ob

    from folx_amd import kernels as K

    print(f'case norm_dense rows={rows} P={P} K={Kd} N={N} act={act}', flush=True)
    rng = np.random.default_rng(23)
    x, J, L = rand(rng, *rows, Kd) + 0.5, rand(rng, P, *rows, Kd), rand(rng, *rows, Kd)
    J = J + 0.3 * rand(rng, P, *rows, 1)  # rows with a mean of their own
    g = (1.0 + 0.3 * rand(rng, Kd)) if affine else None
    be = 0.2 * rand(rng, Kd) if affine else None
    W = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32)
    b = rand(rng, N) if bias else None
    h = ob.layer_norm(ob.OArr(*f64(x, J, L)), None if g is None else g.astype(np.float64),
                      None if be is None else be.astype(np.float64), 1e-5)
    ref = rules.dense_rule(h.x, h.J, h.lap, W.astype(np.float64), None if b is None else b.astype(np.float64))
    if act is not None:
        ref = rules.elementwise_rule(act, *ref)
    assert K.norm_dense_supported(act, Kd, N, int(np.prod(rows)))
    opt = lambda t: None if t is None else dev(t)
    for rep in range(2):  # the workspace of the second call holds what the first one left
        got = K.norm_dense(act, dev(x), dev(J), dev(L), opt(g), opt(be), 1e-5, dev(W), opt(b))
        assert_triplet(got, ref, f'norm_dense call {rep}')


def test_norm_dense_matches_three_kernels_large():
    """A transformer layer's LayerNorm + MLP product at a full chunk: the fused rule and
    layernorm + dense + elementwise agree to rounding."""
    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(7)
    R, P, Kd, N = 256 * 32, 96, 256, 256
    x = torch.randn(R, Kd, device='cuda', generator=g)
    J = torch.randn(P, R, Kd, device='cuda', generator=g)
    L = torch.randn(R, Kd, device='cuda', generator=g)
    gam = 1 + 0.2 * torch.randn(Kd, device='cuda', generator=g)
    bet = 0.2 * torch.randn(Kd, device='cuda', generator=g)
    W = torch.randn(Kd, N, device='cuda', generator=g) / 16
    b = torch.randn(N, device='cuda', generator=g)
    for act in (None, 'tanh'):
        got = K.norm_dense(act, x, J, L, gam, bet, 1e-5, W, b)
        ref = K.dense(*K.layernorm(x, J, L, gam, bet, 1e-5), W, b)
        if act is not None:
            ref = K.elementwise(act, *ref)
        for a, r, nm in zip(got, ref, ('x', 'jac', 'lap')):
            torch.testing.assert_close(a, r, rtol=1e-4 if nm == 'lap' else 2e-5, atol=2e-3 if nm == 'lap' else 2e-5,
                                       msg=lambda m: f'{act} {nm}: {m}')


@pytest.mark.parametrize('B,n,P,widths,bcast,N,act', [
    (4, 16, 48, (256, 256, 256, 32, 32), (0, 1, 1, 0, 0), 256, 'tanh'),   # FermiNet-style one-electron layer
    (2, 6, 30, (16, 32), (1, 0), 132, 'silu'),                            # groups of 32 rows (12 positions), broadcast part first
    (1, 8, 5, (48,), (0,), 300, 'sin'),                                   # a single part
    (3, 8, 17, (16, 16, 16, 16, 16, 16, 16, 16), (0, 1, 0, 1, 0, 1, 0, 1), 256, 'softplus'),  # eight parts
])
def test_dense_act_parts(B, n, P, widths, bcast, N, act):
    """The wide dense + activation rule reading its Jacobian operand part by part equals the
    oracle's rules on the concatenated operand."""
    from folx_amd import kernels as K

    print(f'case dense_act_parts B={B} n={n} P={P} widths={widths} bcast={bcast} N={N}', flush=True)
    rng = np.random.default_rng(29)
    Kd = sum(widths)
    xs, ls, Js, Jd = [], [], [], []
    for w, bc in zip(widths, bcast):
        lead = (B,) if bc else (B, n)
        xp_, lp_, Jp = rand(rng, *lead, w), rand(rng, *lead, w), rand(rng, P, *lead, w)
        Js.append(Jp)
        if bc:
            xp_, lp_, Jp = (np.broadcast_to(np.expand_dims(t, -2), (*t.shape[:-1], n, w)) for t in (xp_, lp_, Jp))
        xs.append(xp_), ls.append(lp_), Jd.append(Jp)
    x, L, J = np.concatenate(xs, -1), np.concatenate(ls, -1), np.concatenate(Jd, -1)
    W = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32)
    b = rand(rng, N)
    ref = rules.elementwise_rule(act, *rules.dense_rule(*f64(x, J, L, W), b.astype(np.float64)))
    for rep in range(2):
        got = K.dense_act_parts(act, dev(x), dev(L), [dev(t) for t in Js], widths, bcast, n, dev(W), dev(b))
        assert_triplet(got, ref, f'dense_act_parts call {rep}')
    # with a skip connection added in the epilogue
    res = (rand(rng, B, n, N), rand(rng, P, B, n, N), rand(rng, B, n, N))
    got = K.dense_act_parts(act, dev(x), dev(L), [dev(t) for t in Js], widths, bcast, n, dev(W), dev(b), 0.0,
                            tuple(dev(t) for t in res))
    assert_triplet(got, tuple(a + r.astype(np.float64) for a, r in zip(ref, res)), 'dense_act_parts + residual')
    # with a per-walker term added in front of the activation (and the skip connection behind it)
    pre = (rand(rng, B, N), rand(rng, P, B, N), rand(rng, B, N))
    z = rules.dense_rule(*f64(x, J, L, W), b.astype(np.float64))
    z = tuple(t + np.expand_dims(q.astype(np.float64), -2) for t, q in zip(z, pre))
    ref = rules.elementwise_rule(act, *z)
    got = K.dense_act_parts(act, dev(x), dev(L), [dev(t) for t in Js], widths, bcast, n, dev(W), dev(b), 0.0, None,
                            tuple(dev(t) for t in pre))
    assert_triplet(got, ref, 'dense_act_parts + pre-activation term')
    got = K.dense_act_parts(act, dev(x), dev(L), [dev(t) for t in Js], widths, bcast, n, dev(W), dev(b), 0.0,
                            tuple(dev(t) for t in res), tuple(dev(t) for t in pre))
    assert_triplet(got, tuple(a + r.astype(np.float64) for a, r in zip(ref, res)), 'dense_act_parts + pre + residual')


def test_norm_dense_full_chunk_properties():
    """At the benchmark's chunk size (32768 positions, 96 Jacobian rows): the fused rule is
    linear in the Jacobian rows up to its quadratic lap term, so doubling them doubles y_jac bit
    for bit (a power of two) and leaves y alone; and every position is computed from its own
    data in a fixed order, so reversing the positions reverses the results bit for bit."""
    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(11)
    R, P, Kd, N = 1024 * 32, 96, 256, 256
    x = torch.randn(R, Kd, device='cuda', generator=g)
    J = torch.randn(P, R, Kd, device='cuda', generator=g)
    L = torch.randn(R, Kd, device='cuda', generator=g)
    gam = 1 + 0.2 * torch.randn(Kd, device='cuda', generator=g)
    bet = 0.2 * torch.randn(Kd, device='cuda', generator=g)
    W = torch.randn(Kd, N, device='cuda', generator=g) / 16
    b = torch.randn(N, device='cuda', generator=g)
    print('case norm_dense full chunk', flush=True)
    y, yj, yl = K.norm_dense('tanh', x, J, L, gam, bet, 1e-5, W, b)
    assert torch.isfinite(yj).all() and torch.isfinite(yl).all()
    J.mul_(2.0)
    y2, yj2, yl2 = K.norm_dense('tanh', x, J, L, gam, bet, 1e-5, W, b)
    assert torch.equal(y2, y)
    yj.mul_(2.0)
    assert torch.equal(yj2, yj)
    del yj
    # positions reversed (J is the doubled one)
    xr, Lr = x.flip(0).contiguous(), L.flip(0).contiguous()
    J = J.flip(1).contiguous()
    y3, yj3, yl3 = K.norm_dense('tanh', xr, J, Lr, gam, bet, 1e-5, W, b)
    assert torch.equal(y3, y2.flip(0)) and torch.equal(yl3, yl2.flip(0))
    assert torch.equal(yj3, yj2.flip(1))


def test_dense_act_parts_full_chunk_equals_concatenated():
    """At the FermiNet-style chunk size (1024 walkers x 16 electrons, 48 Jacobian rows, 832
    features in five parts, two of them per-walker): reading the operand in parts does the
    same arithmetic in the same order as reading the concatenated array, so the results are
    equal bit for bit."""
    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(12)
    B, n, P, N = 1024, 16, 48, 256
    widths, bcast = (256, 256, 256, 32, 32), (0, 1, 1, 0, 0)
    xs, ls, Js, Jd = [], [], [], []
    for w, bc in zip(widths, bcast):
        lead = (B,) if bc else (B, n)
        xp_ = torch.randn(*lead, w, device='cuda', generator=g)
        lp_ = torch.randn(*lead, w, device='cuda', generator=g)
        Jp = torch.randn(P, *lead, w, device='cuda', generator=g)
        Js.append(Jp)
        ex = (lambda t: t.unsqueeze(-2).expand(*t.shape[:-1], n, w)) if bc else (lambda t: t)
        xs.append(ex(xp_)), ls.append(ex(lp_)), Jd.append(ex(Jp))
    x, L, J = torch.cat(xs, -1), torch.cat(ls, -1), torch.cat(Jd, -1)
    W = torch.randn(sum(widths), N, device='cuda', generator=g) / 29
    b = torch.randn(N, device='cuda', generator=g)
    print('case dense_act_parts full chunk', flush=True)
    ref = K.dense_act('tanh', x, J, L, W, b)
    got = K.dense_act_parts('tanh', x, L, Js, widths, bcast, n, W, b)
    for a, r in zip(got, ref):
        assert torch.equal(a, r)
    res = tuple(torch.randn_like(t) for t in ref)
    got = K.dense_act_parts('tanh', x, L, Js, widths, bcast, n, W, b, 0.0, res)
    for a, r, s_ in zip(got, ref, res):
        torch.testing.assert_close(a, r + s_, rtol=2e-6, atol=2e-6)  # the epilogue adds with one rounding (fma)


def test_dense_act_wide_matches_two_kernels_large():
    """A transformer MLP layer at a full chunk: the fused wide path and dense + elementwise
    agree to rounding (the sums over Jacobian rows are taken in a different order)."""
    from folx_amd import kernels as K

    g = torch.Generator(device='cuda').manual_seed(6)
    R, P, Kd, N = 256 * 32, 96, 256, 256
    x = torch.randn(R, Kd, device='cuda', generator=g)
    J = torch.randn(P, R, Kd, device='cuda', generator=g)
    L = torch.randn(R, Kd, device='cuda', generator=g)
    W = torch.randn(Kd, N, device='cuda', generator=g) / 16
    b = torch.randn(N, device='cuda', generator=g)
    assert K.dense_act_supported('tanh', Kd, N, rows=R)
    got = K.dense_act('tanh', x, J, L, W, b)
    ref = K.elementwise('tanh', *K.dense(x, J, L, W, b))
    for a, r, nm in zip(got, ref, ('x', 'jac', 'lap')):
        torch.testing.assert_close(a, r, rtol=1e-4 if nm == 'lap' else 2e-5, atol=1e-3 if nm == 'lap' else 2e-5,
                                   msg=lambda m: f'{nm}: {m}')


@pytest.mark.parametrize('lead,n,lo,hi,P,Kd,N', [((5,), 32, 0, 16, 9, 256, 256), ((5,), 32, 16, 32, 9, 256, 256),
                                                 ((2, 3), 7, 2, 5, 4, 48, 20), ((4,), 9, 1, 9, 3, 17, 33),
                                                 ((300,), 6, 3, 4, 2, 32, 64), ((7,), 6, 1, 5, 3, 40, 1)])
def test_dense_row_slice(lead, n, lo, hi, P, Kd, N):
    """A slice along the axis in front of the feature axis is read in place by the GEMM."""
    from folx_amd import kernels as K

    print(f'case dense row_slice lead={lead} n={n} [{lo}:{hi}] P={P} K={Kd} N={N}', flush=True)
    rng = np.random.default_rng(20)
    x, J, L = rand(rng, *lead, n, Kd), rand(rng, P, *lead, n, Kd), rand(rng, *lead, n, Kd)
    W, b = (rand(rng, Kd, N) / np.sqrt(Kd)).astype(np.float32), rand(rng, N)
    ref = rules.dense_rule(*f64(x[..., lo:hi, :], J[..., lo:hi, :], L[..., lo:hi, :], W), b.astype(np.float64))
    got = K.dense(dev(x), dev(J), dev(L), dev(W), dev(b), None, (lo, hi))
    assert got[0].shape == (*lead, hi - lo, N)
    assert_triplet(got, ref, 'dense row_slice')


def test_dense_linearity_large():
    """Size-independent property at full PsiFormer row counts: the rule is linear, so
    f(a h1 + h2) = a f(h1) + f(h2) row by row, and zero rows map to zero."""
    from folx_amd import kernels as K

    rng = np.random.default_rng(3)
    R, P, Kd, N = 4096 * 8, 10, 256, 256
    g = torch.Generator(device='cuda').manual_seed(0)
    x = torch.randn(R, Kd, device='cuda', generator=g)
    J = torch.randn(P, R, Kd, device='cuda', generator=g)
    L = torch.zeros(R, Kd, device='cuda')
    W = dev(rand(rng, Kd, N) / 16)
    y1, J1, L1 = K.dense(x, J, L, W)
    assert float(L1.abs().max()) == 0.0
    # rows of J are just more rows of the same GEMM: J1[0] must equal dense(J[0]) as x
    y2, _, _ = K.dense(J[0].contiguous(), J[:1].contiguous(), L, W)
    assert torch.equal(y2, J1[0])
    # against an fp64 product on a row sample
    idx = torch.randint(0, R, (64,), device='cuda')
    ref = (x[idx].double() @ W.double()).cpu().numpy()
    assert_val(y1[idx], ref, 'dense sample')


@pytest.mark.parametrize('op', ['mul', 'div', 'add', 'sub'])
@pytest.mark.parametrize('sa,sb', [((3, 4, 6), (3, 4, 6)), ((3, 4, 6), (3, 4, 1)), ((3, 1, 6), (3, 4, 6)),
                                   ((2, 5, 1, 7), (2, 1, 3, 7))])
def test_binary(op, sa, sb):
    from folx_amd import kernels as K

    print(f'case binary {op} {sa} {sb}', flush=True)
    rng = np.random.default_rng(4)
    P = 6
    a, aj, al = rand(rng, *sa), rand(rng, P, *sa), rand(rng, *sa)
    b, bj, bl = rand(rng, *sb), rand(rng, P, *sb), rand(rng, *sb)
    if op == 'div':
        b = np.abs(b) + 0.5
    rule = {'mul': rules.mul_rule, 'div': rules.div_rule, 'add': rules.add_rule,
            'sub': lambda *t: rules.add_rule(*t, sign=-1.0)}[op]
    A = [np.broadcast_to(t, np.broadcast_shapes(t.shape, u.shape)) for t, u in
         zip(f64(a, aj, al), f64(b, bj, bl))]
    Bb = [np.broadcast_to(u, np.broadcast_shapes(t.shape, u.shape)) for t, u in
          zip(f64(a, aj, al), f64(b, bj, bl))]
    ref = rule(*A, *Bb)
    got = K.binary(op, dev(a), dev(aj), dev(al), dev(b), dev(bj), dev(bl))
    assert_triplet(got, ref, op)


def test_rows_affine():
    from folx_amd import kernels as K

    rng = np.random.default_rng(5)
    rows, shape = 5, (3, 4, 6)
    inp = rand(rng, rows, *shape)
    c, d = rand(rng, 3, 1, 6), rand(rng, 1, 4, 1)
    got = K.rows_affine(dev(inp), rows, shape, shape, dev(c), dev(d), alpha=0.5, beta=-2.0)
    assert_val(got, 0.5 * inp.astype(np.float64) * c + (-2.0) * d)
    got = K.rows_affine(dev(inp[:, :, :1]), rows, (3, 1, 6), shape, None, None, alpha=-1.0)
    assert_val(got, -np.broadcast_to(inp[:, :, :1], (rows, *shape)))
    # a coefficient that is broadcast along two inner axes of a four-axis index space (an identity per
    # matrix against (walker, row, determinant, column)): the wrapper spells the broadcast out
    shape4 = (2, 5, 3, 5)
    inp4 = rand(rng, 2, *shape4)
    eye = (7.0 * np.eye(5, dtype=np.float32))[None, :, None, :]
    got = K.rows_affine(dev(inp4), 2, shape4, shape4, None, dev(eye), alpha=1.0, beta=1.0)
    assert_val(got, inp4.astype(np.float64) + eye)
    got = K.rows_affine(dev(inp4[:, :, :, :1]), 2, (2, 5, 1, 5), shape4, dev(eye), None, alpha=2.0)
    assert_val(got, 2.0 * np.broadcast_to(inp4[:, :, :, :1], (2, *shape4)).astype(np.float64) * eye)
    # the INPUT broadcast along two separate groups of axes (what an outer-product style multiply of (n, 1, d, 1) with
    # (n, m, d, e) gives): more than three index dimensions, spelled out in two passes
    shape5 = (2, 5, 4, 8, 8)
    inp5 = rand(rng, 3, 2, 5, 1, 8, 1)
    c5 = rand(rng, 1, 1, 4, 8, 8)
    got = K.rows_affine(dev(inp5), 3, (2, 5, 1, 8, 1), shape5, dev(c5), None, alpha=1.5)
    assert_val(got, 1.5 * np.broadcast_to(inp5, (3, *shape5)).astype(np.float64) * c5)
    got = K.rows_affine(dev(inp5[:, :, :, :, :1]), 3, (2, 5, 1, 1, 1), shape5, None, dev(c5), alpha=1.0, beta=2.0)
    assert_val(got, np.broadcast_to(inp5[:, :, :, :, :1], (3, *shape5)).astype(np.float64) + 2.0 * c5)


@pytest.mark.parametrize('outer,red,inner', [(7, 5, 9), (6, 100, 1), (3, 4, 1), (1, 33, 70)])
def test_reduce(outer, red, inner):
    from folx_amd import kernels as K

    rng = np.random.default_rng(6)
    rows = 4
    inp = rand(rng, rows, outer, red, inner)
    got = K.reduce_sum(dev(inp), rows, outer, red, inner, alpha=0.25)
    assert_val(got, 0.25 * inp.astype(np.float64).sum(2))
    got = K.reduce_max(dev(inp[0]), outer, red, inner)
    assert_val(got, inp[0].max(1))
    # a window of the reduced axis, read in place (empty, inner, trailing, whole)
    for lo, hi in ((0, 0), (1, max(1, red - 1)), (red // 2, red), (0, red)):
        got = K.reduce_sum(dev(inp), rows, outer, red, inner, alpha=2.0, window=(lo, hi))
        assert_val(got, 2.0 * inp.astype(np.float64)[:, :, lo:hi].sum(2))


def test_gather_and_scatter_rows():
    from folx_amd import kernels as K

    rng = np.random.default_rng(7)
    k_in, B, So, Si, k_out = 3, 4, 5, 6, 7
    mask = rng.integers(-1, k_out, size=(k_in, So))
    data = rand(rng, k_in, B, So, Si)
    ref = ia.materialize(data.astype(np.float64), np.broadcast_to(mask[:, :, None], (k_in, So, Si)), k_out)
    # static gather table: slot s of (t, so) = s-th row r with mask[r, so] == t
    n_slots = max(1, int(max((mask[:, so] == t).sum() for so in range(So) for t in range(k_out))))
    take = np.full((k_out, n_slots, So), -1, dtype=np.int32)
    for so in range(So):
        for t in range(k_out):
            rows = np.nonzero(mask[:, so] == t)[0]
            take[t, : len(rows), so] = rows
    got = K.gather_rows(dev(data).reshape(k_in, B, So * Si), dev(take, torch.int32), k_out, n_slots, B, So, Si)
    assert_val(got.reshape(k_out, B, So, Si), ref)
    got = K.scatter_add_rows(dev(data).reshape(k_in, B, So * Si), dev(mask, torch.int32), k_out, B, So, Si)
    assert_val(got.reshape(k_out, B, So, Si), ref)


@pytest.mark.parametrize('collide', [False, True])
@pytest.mark.parametrize('k_in,B,So,Si,k_out', [(3, 4, 5, 6, 7), (3, 2, 32, 256, 96), (6, 3, 17, 1, 9)])
def test_scatter_add_rows_into_existing(collide, k_in, B, So, Si, k_out):
    """``scatter_add_rows(out=existing)``: a sparse Jacobian added in place into a dense row stack that
    already holds values (the sparse skip connection added into a product's fresh output,
    folx/api.py:230-249 through the dense branch).  Non-colliding: every (target row, position) is
    named at most once; colliding: several stored rows of a position name the same target row."""
    from folx_amd import kernels as K

    rng = np.random.default_rng(70 + k_in + So)
    if collide:
        mask = rng.integers(-1, min(k_out, 2), size=(k_in, So))  # targets 0 / 1 only: collisions everywhere
    else:
        mask = np.stack([rng.permutation(k_out)[:k_in] for _ in range(So)], axis=1)  # distinct rows per position
        mask[rng.random(mask.shape) < 0.2] = -1
    data = rand(rng, k_in, B, So, Si)
    base = rand(rng, k_out, B, So, Si)
    ref = base.astype(np.float64) + ia.materialize(data.astype(np.float64),
                                                   np.broadcast_to(mask[:, :, None], (k_in, So, Si)), k_out)
    out = dev(base).reshape(k_out, B, So * Si)
    keep = out.clone()
    got = K.scatter_add_rows(dev(data).reshape(k_in, B, So * Si), dev(mask, torch.int32), k_out, B, So, Si, out=out)
    assert got.data_ptr() == out.data_ptr(), 'accumulates in place'
    assert_val(got.reshape(k_out, B, So, Si), ref)
    # rows that no entry names keep their bits
    named = np.zeros((k_out, So), dtype=bool)
    for r in range(k_in):
        for so in range(So):
            if mask[r, so] >= 0:
                named[mask[r, so], so] = True
    untouched = torch.as_tensor(~named, device=out.device)[:, None, :, None].expand(k_out, B, So, Si)
    assert torch.equal(got.reshape(k_out, B, So, Si)[untouched], keep.reshape(k_out, B, So, Si)[untouched])


@pytest.mark.parametrize('n,P,lead', [(1, 3, (4,)), (2, 5, (3, 2)), (5, 7, (6,)), (8, 24, (4, 3)),
                                      (16, 96, (5, 4)), (32, 20, (3, 2)), (11, 4, (7,)),
                                      # two matrices per wavefront with an odd count; one matrix; a
                                      # workgroup whose last wavefronts have no matrix; rows past a
                                      # multiple of the staging depth
                                      (5, 7, (7,)), (8, 13, (1,)), (16, 19, (9,)), (3, 1, (2, 5))])
def test_slogdet(n, P, lead):
    from folx_amd import kernels as K

    print(f'case slogdet n={n} P={P} lead={lead}', flush=True)
    rng = np.random.default_rng(8)
    A = rand(rng, *lead, n, n)
    J = rand(rng, P, *lead, n, n)
    L = rand(rng, *lead, n, n)
    sign, (ld, jac, lap) = rules.slogdet_rule(*f64(A, J, L))
    gs, gld, gj, gl = K.slogdet(dev(A), dev(J), dev(L))
    np.testing.assert_array_equal(gs.cpu().numpy(), sign)
    # A^-1 amplifies rounding by the condition number: scale the bar with it
    cond = float(np.linalg.cond(A.astype(np.float64)).max())
    amp = max(1.0, cond / 50)
    np.testing.assert_allclose(gld.cpu().numpy(), ld, rtol=1e-5 * amp, atol=1e-6 * amp)
    sc = float(np.abs(jac).max())
    np.testing.assert_allclose(gj.cpu().numpy(), jac, rtol=1e-5 * amp, atol=2e-6 * amp * sc)
    sl = float(np.abs(lap).max())
    np.testing.assert_allclose(gl.cpu().numpy(), lap, rtol=1e-4 * amp, atol=1e-5 * amp * sl)


@pytest.mark.parametrize('outer,mid,n,P', [((3,), (4,), 5, 7), ((2, 2), (16,), 16, 9), ((4,), (3, 2), 8, 5),
                                            ((2,), (1,), 32, 4),
                                            # pairs of 4 x 4 matrices that straddle two batch entries
                                            ((3,), (3,), 4, 6), ((5,), (16,), 8, 48)])
def test_slogdet_row_axis(outer, mid, n, P):
    """Matrices whose rows sit on another axis are read in place: A (*outer, n, *mid, n)."""
    from folx_amd import kernels as K

    print(f'case slogdet row_axis outer={outer} mid={mid} n={n} P={P}', flush=True)
    rng = np.random.default_rng(21)
    shape = (*outer, n, *mid, n)
    ra = len(outer)
    A = (rand(rng, *shape) / np.sqrt(n)).astype(np.float32)
    idx = np.arange(n)
    np.moveaxis(A, ra, -2)[..., idx, idx] += 2.0   # dominant diagonal: well conditioned
    J, L = rand(rng, P, *shape), rand(rng, *shape)
    sign, (ld, jac, lap) = rules.slogdet_rule(*f64(np.moveaxis(A, ra, -2), np.moveaxis(J, ra + 1, -2),
                                                   np.moveaxis(L, ra, -2)))
    gs, gld, gj, gl = K.slogdet(dev(A), dev(J), dev(L), ra)
    np.testing.assert_array_equal(gs.cpu().numpy(), sign)
    assert_val(gld, ld, 'logdet'), assert_val(gj, jac, 'jac'), assert_lap(gl, lap, 'lap')


def test_slogdet_closed_forms_gpu():
    """Well-conditioned closed forms at the strict bar: diagonal matrices and a row swap."""
    from folx_amd import kernels as K

    rng = np.random.default_rng(9)
    B, n, P = 64, 16, 12
    a = (rng.uniform(0.5, 2.0, size=(B, n)) * rng.choice([-1, 1], size=(B, n))).astype(np.float32)
    A = np.zeros((B, n, n), np.float32)
    A[:, range(n), range(n)] = a
    Jd = rand(rng, P, B, n)
    J = np.zeros((P, B, n, n), np.float32)
    J[:, :, range(n), range(n)] = Jd
    Ld = rand(rng, B, n)
    L = np.zeros((B, n, n), np.float32)
    L[:, range(n), range(n)] = Ld
    perm = rng.permutation(n)
    gs, gld, gj, gl = K.slogdet(dev(A[:, perm]), dev(J[:, :, perm]), dev(L[:, perm]))
    a64, Jd64, Ld64 = f64(a, Jd, Ld)
    from math import prod  # noqa: F401

    # sign of the permutation
    inv = sum(1 for i in range(n) for j in range(i + 1, n) if perm[i] > perm[j])
    psign = -1.0 if inv % 2 else 1.0
    np.testing.assert_array_equal(gs.cpu().numpy(), psign * np.prod(np.sign(a64), -1))
    assert_val(gld, np.log(np.abs(a64)).sum(-1), 'logdet')
    assert_val(gj, (Jd64 / a64[None]).sum(-1), 'jac')
    assert_lap(gl, (Ld64 / a64).sum(-1) - ((Jd64 / a64[None]) ** 2).sum((0, -1)), 'lap')


MHSA_CASES = [
    # B, n, H, d, P, valid electrons (None = all)
    (2, 1, 1, 4, 3, None),
    (1, 16, 4, 32, 48, None),    # shape of test_attention.py:320-326
    (1, 16, 4, 32, 48, 4),       # padded sequence (max_sequence = 4)
    (3, 32, 4, 64, 12, None),    # PsiFormer-style tile
    (2, 20, 2, 24, 9, 13),       # sizes that are no multiple of 16
    (1, 64, 2, 64, 6, None),     # large-config tile
]


@pytest.mark.parametrize('B,n,H,d,P,valid', MHSA_CASES)
def test_mhsa(B, n, H, d, P, valid):
    from folx_amd import kernels as K

    print(f'case mhsa B={B} n={n} H={H} d={d} P={P} valid={valid}', flush=True)
    rng = np.random.default_rng(10)
    sig = [1 / np.sqrt(d), 1.0, 1.0]  # q pre-scaled by the caller (test_attention.py:38)
    args = []
    for s in sig:
        args += [s * rand(rng, B, n, H, d), s * rand(rng, P, B, n, H, d), s * rand(rng, B, n, H, d)]
    mask = np.ones((B, n), dtype=bool)
    imask = np.ones((P, B), dtype=bool)
    if valid is not None:
        mask[:, valid:] = False
        imask[min(P, 3 * valid):] = False
    ref = rules.mhsa_rule(*f64(*args), mask, imask)
    got = K.mhsa(*[dev(t) for t in args], dev(mask, torch.uint8), dev(imask, torch.uint8))
    m = mask[0]
    # rows of padding queries carry no meaning (the reference masks them before comparing)
    assert_val(got[0][:, m], ref[0][:, m], 'o')
    assert_val(got[1][:, :, m], ref[1][:, :, m], 'o_jac')
    assert_lap(got[2][:, m], ref[2][:, m], 'o_lap')
    for t in got:
        assert torch.isfinite(t).all()
    if valid is None:
        got2 = K.mhsa(*[dev(t) for t in args], None, None)
        for g1, g2 in zip(got, got2):
            assert torch.equal(g1, g2)


@pytest.mark.parametrize('B,n,H,d,k,missing', [(3, 32, 4, 64, 3, False), (2, 7, 2, 8, 3, True), (1, 64, 1, 64, 3, False),
                                              (2, 16, 2, 32, 6, False), (2, 5, 3, 12, 1, False), (1, 33, 2, 60, 2, True),
                                              (1, 12, 1, 64, 8, False)])
def test_mhsa_sparse(B, n, H, d, k, missing):
    """Attention with position-sparse Jacobians against the dense rule of the oracle on the
    materialised Jacobians, and against the dense kernel."""
    from folx_amd import kernels as K

    print(f'case mhsa_sparse B={B} n={n} H={H} d={d} k={k} missing={missing}', flush=True)
    rng = np.random.default_rng(12)
    index = rng.permutation(n * k).reshape(k, n).astype(np.int32)   # every dense row named once
    P = n * k
    if missing:
        index[k - 1, n // 2] = -1      # an empty slot: its dense row stays zero
        index[0, 0] = -1
    sig = [1 / np.sqrt(d), 1.0, 1.0]
    vals, sparse, laps, dense = [], [], [], []
    for s in sig:
        vals.append(s * rand(rng, B, n, H, d))
        js = s * rand(rng, k, B, n, H, d)
        sparse.append(js)
        laps.append(s * rand(rng, B, n, H, d))
        J = np.zeros((P, B, n, H, d), dtype=np.float32)
        for sl in range(k):
            for e in range(n):
                if index[sl, e] >= 0:
                    J[index[sl, e], :, e] = js[sl, :, e]
        dense.append(J)
    ref = rules.mhsa_rule(*f64(vals[0], dense[0], laps[0], vals[1], dense[1], laps[1], vals[2], dense[2], laps[2]))
    assert K.mhsa_sparse_supported(n, d, k)
    got = K.mhsa_sparse(dev(vals[0]), dev(sparse[0]), dev(laps[0]), dev(vals[1]), dev(sparse[1]), dev(laps[1]),
                        dev(vals[2]), dev(sparse[2]), dev(laps[2]), dev(index, torch.int32), P, not missing)
    assert_val(got[0], ref[0], 'o')
    assert_val(got[1], ref[1], 'o_jac')
    assert_lap(got[2], ref[2], 'o_lap')
    full = K.mhsa(dev(vals[0]), dev(dense[0]), dev(laps[0]), dev(vals[1]), dev(dense[1]), dev(laps[1]),
                  dev(vals[2]), dev(dense[2]), dev(laps[2]), None, None)
    assert_val(got[1], full[1].double().cpu().numpy(), 'o_jac vs dense kernel')
    assert_lap(got[2], full[2].double().cpu().numpy(), 'o_lap vs dense kernel')


@pytest.mark.parametrize('B,shape,P,k', [(3, (5, 7), 12, 3), (2, (16, 256), 96, 3), (1, (4,), 5, 1), (2, (3, 3), 20, 6)])
def test_mul_sparse(B, shape, P, k):
    """Product of a dense-Jacobian triplet with a sparse-Jacobian one against the mul rule on
    the densified operand."""
    from folx_amd import kernels as K

    print(f'case mul_sparse B={B} shape={shape} P={P} k={k}', flush=True)
    rng = np.random.default_rng(22)
    S_w = int(np.prod(shape))
    table = np.stack([rng.permutation(P)[:k] for _ in range(S_w)], 1).astype(np.int32)   # distinct rows per element
    table[rng.uniform(size=table.shape) < 0.15] = -1
    a, aj, al = rand(rng, B, *shape), rand(rng, P, B, *shape), rand(rng, B, *shape)
    b, bj, bl = rand(rng, B, *shape), rand(rng, k, B, *shape), rand(rng, B, *shape)
    dense = np.zeros((P, B, S_w))
    for s_ in range(k):
        for e in range(S_w):
            if table[s_, e] >= 0:
                dense[table[s_, e], :, e] += bj.reshape(k, B, S_w)[s_, :, e]
    ref = rules.mul_rule(*f64(a, aj, al, b), dense.reshape(P, B, *shape), bl.astype(np.float64))
    got = K.mul_sparse(dev(a), dev(aj), dev(al), dev(b), dev(bj), dev(bl), dev(table, torch.int32))
    assert_triplet(got, ref, 'mul_sparse')


@pytest.mark.parametrize('rows,nI,O,P', [((3, 16), 4, 256, 3), ((2, 5), 3, 8, 7), ((1, 1), 1, 4, 0), ((4, 8), 8, 64, 48)])
def test_exp_envelope(rows, nI, O, P):
    """Fused exponential envelope against the chain of primitive rules evaluated by the oracle."""
    from folx_amd import kernels as K
    from oracle import backend as ob

    print(f'case exp_envelope rows={rows} nI={nI} O={O} P={P}', flush=True)
    rng = np.random.default_rng(23)
    d, J, L = np.abs(rand(rng, *rows, nI)) + 0.2, rand(rng, P, *rows, nI), rand(rng, *rows, nI)
    sigma, pi = np.abs(rand(rng, nI, O)) + 0.3, rand(rng, nI, O)
    ref = ob.exp_envelope(ob.OArr(*f64(d, J, L)), sigma.astype(np.float64), pi.astype(np.float64))
    assert K.exp_envelope_supported(nI, O)
    got = K.exp_envelope(dev(d), dev(J), dev(L), dev(sigma), dev(pi))
    assert_triplet(got, (ref.x, ref.J, ref.lap), 'exp_envelope')


@pytest.mark.parametrize('B,ND,n,P,k,strided', [(3, 4, 16, 48, 3, True), (2, 3, 8, 24, 3, True), (2, 2, 5, 9, 2, False),
                                               (1, 16, 16, 96, 3, True), (2, 1, 3, 7, 4, False),
                                               (2, 2, 12, 20, 4, False), (1, 3, 16, 50, 3, False), (2, 2, 7, 11, 1, False)])
def test_slogdet_scaled(B, ND, n, P, k, strided):
    """slogdet of A * F with the product formed on load (sparse Jacobian of F) against the mul
    rule followed by the slogdet rule of the oracle."""
    from folx_amd import kernels as K

    print(f'case slogdet_scaled B={B} ND={ND} n={n} P={P} k={k} strided={strided}', flush=True)
    rng = np.random.default_rng(24)
    shape = (n, ND, n) if strided else (ND, n, n)
    S_w = int(np.prod(shape))
    diag = 1.5 * np.sqrt(n)    # diagonally dominant enough for fp32 at n = 16
    A = rand(rng, B, *shape) + (0 if strided else diag * np.eye(n, dtype=np.float32))
    if strided:
        A = A + diag * np.eye(n, dtype=np.float32)[:, None, :]
    AJ, AL = 0.3 * rand(rng, P, B, *shape), 0.3 * rand(rng, B, *shape)
    F, FJ, FL = 1.0 + 0.2 * rand(rng, B, *shape), 0.3 * rand(rng, k, B, *shape), 0.3 * rand(rng, B, *shape)
    table = np.stack([rng.permutation(P)[:k] for _ in range(S_w)], 1).astype(np.int32)
    table[rng.uniform(size=table.shape) < 0.2] = -1
    dense = np.zeros((P, B, S_w))
    for s_ in range(k):
        for e in range(S_w):
            if table[s_, e] >= 0:
                dense[table[s_, e], :, e] += FJ.reshape(k, B, S_w)[s_, :, e]
    prod = rules.mul_rule(*f64(A, AJ, AL, F), dense.reshape(P, B, *shape), FL.astype(np.float64))
    if strided:
        prod = (np.moveaxis(prod[0], 1, 2), np.moveaxis(prod[1], 2, 3), np.moveaxis(prod[2], 1, 2))
    sign, (ld, jac, lap) = rules.slogdet_rule(*prod)
    got = K.slogdet(dev(A), dev(AJ), dev(AL), 1 if strided else None,
                    (dev(F), dev(FJ), dev(FL), dev(table, torch.int32)))
    np.testing.assert_array_equal(got[0].cpu().numpy(), sign)
    assert_triplet(got[1:], (ld, jac, lap), 'slogdet_scaled')


@pytest.mark.parametrize('rows,F,P', [((3, 5), 8, 4), ((2, 32), 256, 9), ((7,), 512, 3), ((4, 3), 100, 5),
                                      ((2, 2), 1024, 2), ((5,), 4, 1)])
def test_layernorm(rows, F, P):
    """Fused LayerNorm rule against the chain of primitive rules evaluated by the oracle."""
    from folx_amd import kernels as K
    from oracle import backend as ob

    print(f'case layernorm rows={rows} F={F} P={P}', flush=True)
    rng = np.random.default_rng(11)
    x, J, L = rand(rng, *rows, F), rand(rng, P, *rows, F), rand(rng, *rows, F)
    g, b = 1 + 0.1 * rand(rng, F), rand(rng, F)
    ref = ob.layer_norm(ob.OArr(*f64(x, J, L)), g.astype(np.float64), b.astype(np.float64), 1e-5)
    got = K.layernorm(dev(x), dev(J), dev(L), dev(g), dev(b), 1e-5)
    assert_triplet(got, (ref.x, ref.J, ref.lap), 'layernorm')
    got = K.layernorm(dev(x), dev(J), dev(L), None, None, 1e-5)
    ref = ob.layer_norm(ob.OArr(*f64(x, J, L)), None, None, 1e-5)
    assert_triplet(got, (ref.x, ref.J, ref.lap), 'layernorm no affine')


@pytest.mark.parametrize('rows,P,Kd,N', [((3, 32), 7, 256, 256),   # full tiles only: the unchecked epilogue
                                         ((3, 50), 5, 48, 100),    # ragged rows and columns, direct-to-LDS loads
                                         ((2, 9), 3, 20, 36),      # register-staged fallback (K % 16 != 0)
                                         ((4, 11), 6, 100, 1)])    # matrix-vector kernel (N = 1)
def test_dense_residual_epilogue(rows, P, Kd, N):
    from folx_amd import kernels as K

    print(f'case dense residual rows={rows} P={P} K={Kd} N={N}', flush=True)
    rng = np.random.default_rng(12)
    x, J, L = rand(rng, *rows, Kd), rand(rng, P, *rows, Kd), rand(rng, *rows, Kd)
    rx, rJ, rL = rand(rng, *rows, N), rand(rng, P, *rows, N), rand(rng, *rows, N)
    W, b = rand(rng, Kd, N) / 16, rand(rng, N)
    ref = rules.dense_rule(*f64(x, J, L, W), b.astype(np.float64))
    ref = tuple(r + s for r, s in zip(ref, f64(rx, rJ, rL)))
    got = K.dense(dev(x), dev(J), dev(L), dev(W), dev(b), (dev(rx), dev(rJ), dev(rL)))
    assert_triplet(got, ref, 'dense + residual')


@pytest.mark.parametrize('B,n,H,d,P,valid', [(2, 1, 1, 4, 3, None), (1, 16, 4, 32, 48, None), (1, 16, 4, 32, 48, 4),
                                             (2, 32, 4, 64, 12, None), (2, 20, 2, 24, 9, 13)])
def test_mhsea(B, n, H, d, P, valid):
    """Edge-bias attention (shapes of test_attention.py:389-395)."""
    from folx_amd import kernels as K

    print(f'case mhsea B={B} n={n} H={H} d={d} P={P} valid={valid}', flush=True)
    rng = np.random.default_rng(13)
    args = []
    for s in [1 / np.sqrt(d), 1.0, 1.0]:
        args += [s * rand(rng, B, n, H, d), s * rand(rng, P, B, n, H, d), s * rand(rng, B, n, H, d)]
    edge = [rand(rng, B, n, H, n), rand(rng, P, B, n, H, n), rand(rng, B, n, H, n)]
    mask = np.ones((B, n), dtype=bool)
    imask = np.ones((P, B), dtype=bool)
    if valid is not None:
        mask[:, valid:] = False
        imask[min(P, 3 * valid):] = False
    ref = rules.mhsa_rule(*f64(*args), mask, imask, *f64(*edge))
    got = K.mhsa(*[dev(t) for t in args], dev(mask, torch.uint8), dev(imask, torch.uint8), tuple(dev(t) for t in edge))
    m = mask[0]
    assert_val(got[0][:, m], ref[0][:, m], 'o')
    assert_val(got[1][:, :, m], ref[1][:, :, m], 'o_jac')
    assert_lap(got[2][:, m], ref[2][:, m], 'o_lap')


@pytest.mark.parametrize('k_in,k_out,n_slots,B,O,RED,IV,IC', [
    (6, 48, 8, 5, 16, 16, 1, 32),     # pair stream of a FermiNet-style layer: sum over the second electron
    (3, 7, 2, 9, 4, 5, 3, 1),         # table varies along an axis behind the reduced one, scalar tail
    (2, 2, 1, 3, 1, 7, 1, 6),         # tail not a multiple of four
    (4, 5, 11, 2, 3, 4, 2, 8),        # more slots than the kernel keeps in registers
])
def test_gather_reduce_rows(k_in, k_out, n_slots, B, O, RED, IV, IC):
    """Re-indexing with the sum over an axis folded in, data read in its own layout."""
    from folx_amd import kernels as K

    print(f'case gather_reduce_rows {(k_in, k_out, n_slots, B, O, RED, IV, IC)}', flush=True)
    rng = np.random.default_rng(31)
    data = rand(rng, k_in, B, O, RED, IV, IC)
    take = rng.integers(-1, k_in * RED, size=(k_out, n_slots, O, IV)).astype(np.int32)
    ref = np.zeros((k_out, B, O, IV, IC))
    d64 = data.astype(np.float64)
    for t in range(k_out):
        for s in range(n_slots):
            for o in range(O):
                for iv in range(IV):
                    e = take[t, s, o, iv]
                    if e >= 0:
                        ref[t, :, o, iv] += d64[e // RED, :, o, e % RED, iv]
    got = K.gather_reduce_rows(dev(data), dev(take.reshape(k_out, n_slots, O * IV), torch.int32), k_out, n_slots, B, O, RED,
                               IV, IC, 0.125)
    assert_val(got.reshape(ref.shape), 0.125 * ref)

"""Synthetic workloads of the benchmark configurations, written against an operator
namespace ``xp`` (``folx_amd.numpy`` by default) so that the identical model definition
can be evaluated by other back ends that expose the same functions.  The models use plain
calls only (``dot``, ``add``, ``tanh``, ``getitem``, ``mean``, ``concatenate``, ``multiply``,
``transpose``, ``slogdet`` ...): which of them run as one fused rule is the front end's business.

Weights are seeded ``numpy.random.default_rng`` draws with variance ``1 / fan_in``
(lecun-normal-like) and zero biases; positions are per-walker arrays without the walker
axis, as inside ``jax.vmap``.
"""

from __future__ import annotations

import math
from dataclasses import dataclass, field

import numpy as np


def _dense_init(rng, fan_in, fan_out, scale=1.0):
    return (scale * rng.normal(size=(fan_in, fan_out)) / math.sqrt(fan_in)).astype(np.float32)


# --------------------------------------------------------------------------------------
# Node-wise MLP of the reference README (README.md:41-70): 10 x [Dense(100) + SiLU],
# Dense(1), sum.  Input (nodes, 4).
# --------------------------------------------------------------------------------------


def mlp_params(seed=0, in_dim=4, width=100, n_hidden=10):
    rng = np.random.default_rng(seed)
    dims = [in_dim] + [width] * n_hidden + [1]
    return [(_dense_init(rng, a, b), np.zeros(b, np.float32)) for a, b in zip(dims[:-1], dims[1:])]


def mlp_forward(params, x, xp=None):
    if xp is None:
        from . import numpy as xp
    for W, b in params[:-1]:
        x = xp.silu(xp.add(xp.dot(x, W), b))
    W, b = params[-1]
    return xp.sum(xp.add(xp.dot(x, W), b))


# --------------------------------------------------------------------------------------
# PsiFormer-style wavefunction: self-attention layers over electrons, determinants with
# exponential envelopes, log|sum_k det_up det_down|.
# --------------------------------------------------------------------------------------


@dataclass
class PsiFormerConfig:
    n_elec: int = 32
    n_nuc: int = 4
    n_layers: int = 4
    n_heads: int = 4
    head_dim: int = 64
    width: int = 256
    mlp_width: int = 256
    n_det: int = 16
    nuc_box: float = 2.0
    seed: int = 0
    ln_eps: float = 1e-5
    orb_shift: float = 0.0  # c > 0: orbital matrices are A + c I (well-conditioned determinants for parity tests)

    @property
    def n_up(self):
        return self.n_elec // 2

    @property
    def n_down(self):
        return self.n_elec - self.n_up


@dataclass
class PsiFormerParams:
    cfg: PsiFormerConfig
    nuclei: np.ndarray
    spin: np.ndarray
    w_in: np.ndarray
    layers: list = field(default_factory=list)
    w_orb: tuple = ()
    env_sigma: tuple = ()
    env_pi: tuple = ()


def psiformer_params(cfg: PsiFormerConfig) -> PsiFormerParams:
    rng = np.random.default_rng(cfg.seed)
    nuclei = np.random.default_rng(cfg.seed + 1).uniform(-cfg.nuc_box, cfg.nuc_box, size=(cfg.n_nuc, 3)).astype(np.float32)
    n_feat = 4 * cfg.n_nuc + 1
    hd = cfg.n_heads * cfg.head_dim
    p = PsiFormerParams(
        cfg=cfg,
        nuclei=nuclei,
        spin=np.concatenate([np.ones((cfg.n_up, 1)), -np.ones((cfg.n_down, 1))]).astype(np.float32),
        w_in=_dense_init(rng, n_feat, cfg.width),
    )
    for _ in range(cfg.n_layers):
        p.layers.append(
            dict(
                ln1_g=np.ones(cfg.width, np.float32), ln1_b=np.zeros(cfg.width, np.float32),
                # the 1/sqrt(d) of scaled-dot-product attention is folded into w_q by the caller
                w_q=_dense_init(rng, cfg.width, hd, 1.0 / math.sqrt(cfg.head_dim)),
                w_k=_dense_init(rng, cfg.width, hd),
                w_v=_dense_init(rng, cfg.width, hd),
                w_o=_dense_init(rng, hd, cfg.width),
                ln2_g=np.ones(cfg.width, np.float32), ln2_b=np.zeros(cfg.width, np.float32),
                w_1=_dense_init(rng, cfg.width, cfg.mlp_width), b_1=np.zeros(cfg.mlp_width, np.float32),
                w_2=_dense_init(rng, cfg.mlp_width, cfg.width), b_2=np.zeros(cfg.width, np.float32),
            )
        )
    p.w_orb = (
        _dense_init(rng, cfg.width, cfg.n_det * cfg.n_up),
        _dense_init(rng, cfg.width, cfg.n_det * cfg.n_down),
    )
    p.env_sigma = tuple(
        rng.uniform(0.5, 1.5, size=(cfg.n_nuc, cfg.n_det * m)).astype(np.float32) for m in (cfg.n_up, cfg.n_down)
    )
    p.env_pi = tuple(
        rng.uniform(0.5, 1.5, size=(cfg.n_nuc, cfg.n_det * m)).astype(np.float32) for m in (cfg.n_up, cfg.n_down)
    )
    return p


def to_device(params, device):
    """Move every weight array of a parameter object (dataclass / dict / list / tuple) to
    ``device`` as float32 torch tensors, once, so that no call re-uploads them."""
    import dataclasses

    import torch

    def conv(v):
        if isinstance(v, np.ndarray) and v.dtype.kind == 'f':
            return torch.as_tensor(v, dtype=torch.float32).to(device)
        if isinstance(v, dict):
            return {k: conv(x) for k, x in v.items()}
        if isinstance(v, (list, tuple)):
            return type(v)(conv(x) for x in v)
        if dataclasses.is_dataclass(v) and not isinstance(v, type) and not type(v).__name__.endswith('Config'):
            return dataclasses.replace(v, **{f.name: conv(getattr(v, f.name)) for f in dataclasses.fields(v)})
        return v

    return conv(params)


def layer_norm_primitives(xp, h, g, b, eps):
    """LayerNorm over the feature axis from primitives (what flax's LayerNorm lowers to)."""
    mu = xp.mean(h, axis=-1, keepdims=True)
    c = xp.subtract(h, mu)
    var = xp.mean(xp.square(c), axis=-1, keepdims=True)
    y = xp.multiply(c, xp.rsqrt(xp.add(var, eps)))
    return xp.add(xp.multiply(y, g), b)


def layer_norm(xp, h, g, b, eps):
    return xp.layer_norm(h, g, b, eps)


def electron_nuclear_features(xp, r, nuclei):
    """r (n, 3) -> d (n, nuc, 3) = r_i - R_I and dist (n, nuc) = |d|."""
    n = r.shape[0] if hasattr(r, 'shape') else len(r)
    d = xp.subtract(xp.expand_dims(r, 1), nuclei)
    dist = xp.sqrt(xp.sum(xp.square(d), axis=-1))
    return d, dist


def psiformer_forward(p: PsiFormerParams, r, xp=None):
    """log|psi(r)| for one walker; r (n_elec, 3)."""
    if xp is None:
        from . import numpy as xp
    cfg = p.cfg
    n, H, dh = cfg.n_elec, cfg.n_heads, cfg.head_dim
    d, dist = electron_nuclear_features(xp, r, p.nuclei)
    feats = xp.concatenate([xp.reshape(d, (n, 3 * cfg.n_nuc)), dist, p.spin], axis=-1)
    h = xp.dot(feats, p.w_in)
    for L in p.layers:
        hn = xp.layer_norm(h, L['ln1_g'], L['ln1_b'], cfg.ln_eps)
        q = xp.reshape(xp.dot(hn, L['w_q']), (n, H, dh))
        k = xp.reshape(xp.dot(hn, L['w_k']), (n, H, dh))
        v = xp.reshape(xp.dot(hn, L['w_v']), (n, H, dh))
        att = xp.multi_head_self_attention(q, k, v)
        h = xp.add(h, xp.dot(xp.reshape(att, (n, H * dh)), L['w_o']))
        hn = xp.layer_norm(h, L['ln2_g'], L['ln2_b'], cfg.ln_eps)
        mlp = xp.tanh(xp.add(xp.dot(hn, L['w_1']), L['b_1']))
        h = xp.add(h, xp.add(xp.dot(mlp, L['w_2']), L['b_2']))
    return log_psi_from_orbitals(xp, cfg, p, h, dist)


def log_psi_from_orbitals(xp, cfg, p, h, dist):
    """log|sum_k det(orbitals_k^up) det(orbitals_k^down)| from the one-electron stream ``h (n, width)``
    and the electron-nucleus distances ``dist (n, n_nuc)``: orbitals = (h @ w_orb) * envelopes."""
    n = cfg.n_elec
    logdets, signs = [], []
    for s, (lo, hi) in enumerate([(0, cfg.n_up), (cfg.n_up, n)]):
        m = hi - lo
        if m == 0:
            continue
        orb = xp.dot(xp.getitem(h, (slice(lo, hi),)), p.w_orb[s])                                # (m, n_det * m)
        env = xp.exp_envelope(xp.getitem(dist, (slice(lo, hi),)), p.env_sigma[s], p.env_pi[s])  # (m, n_det * m)
        # (electron, determinant, orbital) -> one (m x m) matrix per determinant
        mats = xp.multiply(xp.reshape(orb, (m, cfg.n_det, m)), xp.reshape(env, (m, cfg.n_det, m)))
        if cfg.orb_shift:
            mats = xp.add(mats, (cfg.orb_shift * np.eye(m, dtype=np.float32))[:, None, :])
        sg, ld = xp.slogdet(xp.transpose(mats, (1, 0, 2)))
        logdets.append(ld), signs.append(sg)
    total = logdets[0] if len(logdets) == 1 else xp.add(logdets[0], logdets[1])
    sign = signs[0] if len(signs) == 1 else xp.multiply(signs[0], signs[1])
    logpsi, _ = xp.logsumexp(total, axis=0, b=sign)
    return logpsi


# --------------------------------------------------------------------------------------
# FermiNet-style wavefunction: one-electron stream (width w1) and two-electron stream
# (width w2), tanh layers with residual connections, determinants with exponential
# envelopes.  The two-electron stream depends on six coordinates per pair, so it stays a
# sparse Jacobian (k = 6) with ForwardLaplacianOperator(6); the one-electron stream turns
# dense in the first layer through the spin-wise means over electrons.
# --------------------------------------------------------------------------------------


@dataclass
class FermiNetConfig:
    n_elec: int = 16
    n_nuc: int = 4
    n_layers: int = 4
    w1: int = 256
    w2: int = 32
    n_det: int = 16
    nuc_box: float = 2.0
    seed: int = 0
    orb_shift: float = 0.0  # as in PsiFormerConfig

    @property
    def n_up(self):
        return self.n_elec // 2

    @property
    def n_down(self):
        return self.n_elec - self.n_up


@dataclass
class FermiNetParams:
    cfg: FermiNetConfig
    nuclei: np.ndarray
    eye: np.ndarray
    layers: list = field(default_factory=list)
    w_orb: tuple = ()
    env_sigma: tuple = ()
    env_pi: tuple = ()


def ferminet_params(cfg: FermiNetConfig) -> FermiNetParams:
    rng = np.random.default_rng(cfg.seed)
    nuclei = np.random.default_rng(cfg.seed + 1).uniform(-cfg.nuc_box, cfg.nuc_box, size=(cfg.n_nuc, 3)).astype(np.float32)
    p = FermiNetParams(cfg=cfg, nuclei=nuclei, eye=np.eye(cfg.n_elec, dtype=np.float32))
    d1, d2 = 4 * cfg.n_nuc, 4
    for layer in range(cfg.n_layers):
        f_in = 3 * d1 + 2 * d2
        L = dict(v=_dense_init(rng, f_in, cfg.w1), b=np.zeros(cfg.w1, np.float32))
        if layer < cfg.n_layers - 1:  # the last layer does not update the pair stream
            L['w'] = _dense_init(rng, d2, cfg.w2)
            L['c'] = np.zeros(cfg.w2, np.float32)
        p.layers.append(L)
        d1, d2 = cfg.w1, cfg.w2
    p.w_orb = (_dense_init(rng, cfg.w1, cfg.n_det * cfg.n_up), _dense_init(rng, cfg.w1, cfg.n_det * cfg.n_down))
    p.env_sigma = tuple(
        rng.uniform(0.5, 1.5, size=(cfg.n_nuc, cfg.n_det * m)).astype(np.float32) for m in (cfg.n_up, cfg.n_down)
    )
    p.env_pi = tuple(
        rng.uniform(0.5, 1.5, size=(cfg.n_nuc, cfg.n_det * m)).astype(np.float32) for m in (cfg.n_up, cfg.n_down)
    )
    return p


def ferminet_forward(p: FermiNetParams, r, xp=None):
    """log|psi(r)| for one walker; r (n_elec, 3)."""
    if xp is None:
        from . import numpy as xp
    cfg = p.cfg
    n, nu = cfg.n_elec, cfg.n_up
    d, dist = electron_nuclear_features(xp, r, p.nuclei)
    h = xp.concatenate([xp.reshape(d, (n, 3 * cfg.n_nuc)), dist], axis=-1)  # (n, 4 nuc)
    # pair features; the distance of an electron to itself is regularised as in FermiNet:
    # |r_ij + eye| * (1 - eye), so the square root is never taken at zero
    rij = xp.subtract(xp.expand_dims(r, 1), xp.expand_dims(r, 0))  # (n, n, 3)
    r2 = xp.add(xp.sum(xp.square(rij), axis=-1), p.eye)
    rn = xp.multiply(xp.sqrt(r2), 1.0 - p.eye)
    g = xp.concatenate([rij, xp.expand_dims(rn, 2)], axis=-1)  # (n, n, 4)

    up, dn = slice(0, nu), slice(nu, n)
    for li, L in enumerate(p.layers):
        # means over the electrons of one spin, (d1,) each, and over the second electron of every pair, (n, d2)
        hu, hd = xp.mean(xp.getitem(h, (up,)), axis=0), xp.mean(xp.getitem(h, (dn,)), axis=0)
        gu, gd = xp.mean(xp.getitem(g, (slice(None), up)), axis=1), xp.mean(xp.getitem(g, (slice(None), dn)), axis=1)
        d1 = h.shape[-1]
        f = xp.concatenate([h, xp.broadcast_to(hu, (n, d1)), xp.broadcast_to(hd, (n, d1)), gu, gd], axis=-1)
        hn = xp.tanh(xp.add(xp.dot(f, L['v']), L['b']))
        h = xp.add(h, hn) if L['v'].shape[1] == d1 else hn  # residual layer where the widths match
        if 'w' in L:
            gn = xp.tanh(xp.add(xp.dot(g, L['w']), L['c']))
            g = xp.add(g, gn) if gn.shape == g.shape else gn
    return log_psi_from_orbitals(xp, cfg, p, h, dist)


def sample_electrons(n_walkers, n_elec, sigma, seed):
    return (sigma * np.random.default_rng(seed).normal(size=(n_walkers, n_elec, 3))).astype(np.float32)


@dataclass
class MLPConfig:
    """Node-wise MLP of the reference README: input (n_nodes, in_dim) per walker."""

    n_nodes: int = 100
    in_dim: int = 4
    width: int = 100
    n_hidden: int = 10
    seed: int = 0


def sample_inputs(name, n_walkers, seed=2):
    """Seeded synthetic inputs (B, *shape) of a named configuration."""
    cfg, _, sigma, _ = CONFIGS[name]
    if isinstance(cfg, MLPConfig):
        return np.random.default_rng(seed).normal(size=(n_walkers, cfg.n_nodes, cfg.in_dim)).astype(np.float32)
    return sample_electrons(n_walkers, cfg.n_elec, sigma, seed)


def build(name):
    """(forward(params, r, xp=None), params, config, walkers, sigma, threshold) of a named
    benchmark configuration."""
    cfg, walkers, sigma, thr = CONFIGS[name]
    if isinstance(cfg, MLPConfig):
        params = mlp_params(cfg.seed, cfg.in_dim, cfg.width, cfg.n_hidden)
        return mlp_forward, params, cfg, walkers, sigma, thr
    if isinstance(cfg, FermiNetConfig):
        return ferminet_forward, ferminet_params(cfg), cfg, walkers, sigma, thr
    return psiformer_forward, psiformer_params(cfg), cfg, walkers, sigma, thr


CONFIGS = {
    # name: (config, walkers, position sigma, sparsity threshold)
    'mlp_dense': (MLPConfig(), 20, 1.0, 0),     # README.md:63-65, ForwardLaplacianOperator(0)
    'mlp_sparse': (MLPConfig(), 256, 1.0, 4),   # README.md:68-70 model, ForwardLaplacianOperator(4)
    'ferminet16': (FermiNetConfig(), 4096, 1.5, 6),
    'psiformer32': (PsiFormerConfig(), 4096, 1.5, 6),
    'psiformer64': (
        PsiFormerConfig(n_elec=64, n_nuc=8, n_heads=8, head_dim=64, width=512, mlp_width=512, nuc_box=4.0),
        1024, 2.0, 6,
    ),
}

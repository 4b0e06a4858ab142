"""Models written with plain torch (one sample in), for the traced front door: each entry builds ``(fn, x)`` for a
dtype -- float32 for the forward-Laplacian run, float64 for the Hessian trace by torch AD of the SAME function."""

import copy

import numpy as np
import torch
import torch.nn as nn


def _module(make, seed):
    torch.manual_seed(seed)
    m32 = make()
    for p in m32.parameters():
        p.requires_grad_(False)
    return {torch.float32: m32, torch.float64: copy.deepcopy(m32).double()}


def readme_mlp():
    """The README's node-wise MLP (README.md:41-70) as torch modules: 6 nodes x 4 inputs, Dense + SiLU layers, summed."""
    nets = _module(lambda: nn.Sequential(nn.Linear(4, 8), nn.SiLU(), nn.Linear(8, 8), nn.SiLU(), nn.Linear(8, 1)), 0)
    x = np.random.default_rng(0).normal(size=(3, 6, 4)).astype(np.float32)
    return (lambda dt: (lambda t: nets[dt](t).sum())), x


def transformer_block():
    """LayerNorm, per-head attention from matmul / softmax, an MLP with GELU, skip connections, a log-determinant."""
    n, d, H = 5, 8, 2
    mods = _module(lambda: nn.ModuleDict(dict(
        emb=nn.Linear(3, d), ln1=nn.LayerNorm(d), q=nn.Linear(d, d, bias=False), k=nn.Linear(d, d, bias=False),
        v=nn.Linear(d, d, bias=False), o=nn.Linear(d, d), ln2=nn.LayerNorm(d), up=nn.Linear(d, 2 * d),
        down=nn.Linear(2 * d, d), orb=nn.Linear(d, n))), 1)

    def make(dt):
        m = mods[dt]

        def f(x):  # x (n, 3)
            h = torch.tanh(m['emb'](x))
            hn = m['ln1'](h)
            q, k, v = (m[t](hn).view(n, H, d // H).permute(1, 0, 2) for t in ('q', 'k', 'v'))
            p = torch.softmax(q @ k.transpose(-1, -2) / (d // H) ** 0.5, dim=-1)
            h = h + m['o']((p @ v).permute(1, 0, 2).reshape(n, d))
            h = h + m['down'](torch.nn.functional.gelu(m['up'](m['ln2'](h))))
            orbitals = m['orb'](h) + 2.0 * torch.eye(n, dtype=x.dtype)
            sign, logdet = torch.linalg.slogdet(orbitals)
            return logdet + torch.log(torch.cosh(h)).mean()

        return f

    x = (0.6 * np.random.default_rng(1).normal(size=(2, n, 3))).astype(np.float32)
    return make, x


def indexing_and_piecewise():
    """Slices, integer indexing, where / comparisons, clamp, pow, cat / stack, reductions with keepdim, several outputs."""
    w = torch.tensor(np.linspace(-1.0, 1.0, 12).reshape(4, 3))

    def make(dt):
        wd = w.to(dt)

        def f(x):  # x (4, 3)
            a = torch.where(x > 0.1, torch.sin(x), 0.3 * torch.cos(x))
            b = torch.clamp(x * wd, -0.4, 0.6) + x[:, 1:2] ** 3
            c = torch.cat([x[1:3], x[[0, 3]]], dim=0) * torch.exp(-x ** 2).sum(dim=-1, keepdim=True)
            s = torch.stack([a.mean(dim=0), b.amax(dim=0), c.prod(dim=0)], dim=0)
            return s, torch.logsumexp(a + b, dim=-1), (c - c.mean()) / torch.sqrt(c.var(unbiased=False) + 1.0)

        return f

    x = np.random.default_rng(2).normal(size=(3, 4, 3)).astype(np.float32)
    return make, x


def attention_by_name():
    """Attention through the named function (one equation in the trace, the attention rule's kernel) next to
    ``scaled_dot_product_attention`` (traced into products and a softmax), both behind linear maps."""
    from folx_amd.fx import multi_head_self_attention

    n, H, d = 8, 2, 8
    mods = _module(lambda: nn.ModuleDict(dict(emb=nn.Linear(3, H * d), q=nn.Linear(H * d, H * d), k=nn.Linear(H * d, H * d),
                                              v=nn.Linear(H * d, H * d), o=nn.Linear(H * d, 4))), 4)

    def make(dt):
        m = mods[dt]

        def f(x):  # x (n, 3)
            h = torch.tanh(m['emb'](x))
            q, k, v = (m[t](h).view(n, H, d) for t in ('q', 'k', 'v'))
            a = multi_head_self_attention(q * d ** -0.5, k, v).reshape(n, H * d)
            b = torch.nn.functional.scaled_dot_product_attention(q.permute(1, 0, 2), k.permute(1, 0, 2), v.permute(1, 0, 2))
            return m['o'](a + b.permute(1, 0, 2).reshape(n, H * d)).sum(dim=0)

        return f

    x = (0.7 * np.random.default_rng(4).normal(size=(2, n, 3))).astype(np.float32)
    return make, x


MODELS = {'attention_by_name': attention_by_name, 'readme_mlp': readme_mlp, 'transformer_block': transformer_block, 'indexing_and_piecewise': indexing_and_piecewise}

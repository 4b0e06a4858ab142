"""Everyday torch constructs (functional calls, modules, linalg, indexing) as small one-sample functions, for the traced
front door: ``CONSTRUCTS[name] = (make, x)`` with ``make(dtype) -> (fn, fn_for_ad)``.  ``fn_for_ad`` is the same function
spelled so that torch's own second-order AD can differentiate it (fused attention and ``cdist`` have no forward-mode
formula in torch; they are written out for the check)."""

import copy
import types

import numpy as np
import torch
import torch.nn as nn
import torch.nn.functional as F

N, D = 5, 8


def _mods():
    torch.manual_seed(0)
    m32 = types.SimpleNamespace(lin=nn.Linear(3, D), lin2=nn.Linear(D, D), ln=nn.LayerNorm(D),
                                mha=nn.MultiheadAttention(D, 2, batch_first=True), bil=nn.Bilinear(D, D, 4),
                                emb=nn.Embedding(6, D), conv=nn.Conv1d(3, 4, 3, padding=1), gru=nn.GRUCell(3, D))
    for mod in vars(m32).values():
        mod.eval()
        for p in mod.parameters():
            p.requires_grad_(False)
    m64 = types.SimpleNamespace(**{k: copy.deepcopy(v).double() for k, v in vars(m32).items()})
    return {torch.float32: m32, torch.float64: m64}


_M = _mods()


def _heads(t):      # (N, D) -> (1, 2, N, D / 2)
    return t.reshape(1, N, 2, D // 2).transpose(1, 2)


def _attention_by_hand(q, k, v, mask=None, causal=False):
    s = q @ k.transpose(-1, -2) / np.sqrt(q.shape[-1])
    if causal:
        s = s.masked_fill(~torch.tril(torch.ones(s.shape[-2:], dtype=torch.bool)), -1e30)
    if mask is not None:
        s = s.masked_fill(~mask, -1e30) if mask.dtype == torch.bool else s + mask
    return torch.softmax(s, -1) @ v


def _mha_by_hand(m, h):
    w, b = m.mha.in_proj_weight, m.mha.in_proj_bias
    q, k, v = (h @ w[i * D:(i + 1) * D].T + b[i * D:(i + 1) * D] for i in range(3))
    o = _attention_by_hand(_heads(q), _heads(k), _heads(v)).transpose(1, 2).reshape(N, D)
    return m.mha.out_proj(o)


_KEEP = torch.tensor(np.random.default_rng(1).random((N, N)) > 0.3) | torch.eye(N, dtype=torch.bool)
_IDX = torch.tensor([[0, 1], [2, 3], [1, 1], [7, 0], [5, 6]])


def _in_place(lin):
    def f(x):           # updates in place, through views, by slice and by integer arrays
        h = lin(x).clone()
        h += 1.0
        h.mul_(0.5)
        h.tanh_()
        h[:, :2] = x[:, :2] * 2
        h[0] = h[1] * h[2]
        h[torch.tensor([1, 3]), torch.tensor([4, 5])] = x[:2, 0]
        out = torch.zeros(N, 4, dtype=x.dtype)
        out[:, :3] = torch.sin(x)
        out[:, 3] = x.square().sum(-1)
        return h.sum(0)[:4] + out.sum(0)

    def g(x):           # the same values without a single update
        h = torch.tanh((lin(x) + 1.0) * 0.5)
        h = torch.cat([x[:, :2] * 2, h[:, 2:]], 1)
        h = torch.cat([(h[1] * h[2])[None], h[1:]], 0)
        keep = torch.ones(N, D, dtype=x.dtype)
        keep[1, 4] = keep[3, 5] = 0.0
        put = torch.zeros(N, D, dtype=x.dtype)
        e14, e35 = torch.zeros(N, D, dtype=x.dtype), torch.zeros(N, D, dtype=x.dtype)
        e14[1, 4], e35[3, 5] = 1.0, 1.0
        h = h * keep + e14 * x[0, 0] + e35 * x[1, 0] + put
        out = torch.cat([torch.sin(x), x.square().sum(-1, keepdim=True)], 1)
        return h.sum(0)[:4] + out.sum(0)

    return f, g


def _cases(m, dt):
    lin, lin2, ln = m.lin, m.lin2, m.ln
    eye = lambda n, *a: torch.eye(n, *a, dtype=dt)     # noqa: E731
    ones = lambda *s: torch.ones(*s, dtype=dt)         # noqa: E731
    qkv = lambda x: (_heads(lin(x)), _heads(lin(x * 0.5)), _heads(lin(x + 1)))     # noqa: E731
    return {
        'sdpa': (lambda x: F.scaled_dot_product_attention(*qkv(x)).square().sum(),
                 lambda x: _attention_by_hand(*qkv(x)).square().sum()),
        'sdpa_causal': (lambda x: F.scaled_dot_product_attention(*qkv(x), is_causal=True).square().sum(),
                        lambda x: _attention_by_hand(*qkv(x), causal=True).square().sum()),
        'sdpa_bool_mask': (lambda x: F.scaled_dot_product_attention(*qkv(x), attn_mask=_KEEP).square().sum(),
                           lambda x: _attention_by_hand(*qkv(x), mask=_KEEP).square().sum()),
        'mha_module': (lambda x: m.mha(lin(x)[None], lin(x)[None], lin(x)[None], need_weights=False)[0].square().sum(),
                       lambda x: _mha_by_hand(m, lin(x)).square().sum()),
        'cdist': (lambda x: torch.cdist(x, x * 0.5 + 0.1).sum(),
                  lambda x: (x[:, None] - (x * 0.5 + 0.1)[None]).square().sum(-1).sqrt().sum()),
        'normalize': lambda x: F.normalize(lin(x), dim=-1).sum(0),
        'pairwise_norm': lambda x: torch.linalg.norm(x[:, None] - x[None] + eye(N)[..., None], dim=-1).sum(0),
        'vector_norms': lambda x: torch.linalg.vector_norm(lin(x), dim=-1) + torch.linalg.vector_norm(lin(x), 1, dim=-1)
        + torch.linalg.vector_norm(lin(x), float('inf'), dim=-1) + torch.linalg.vector_norm(lin(x), 3, dim=-1),
        'activations': lambda x: (F.softplus(lin(x)) * F.gelu(lin(x)) + F.silu(lin(x)) + F.mish(lin(x)) + F.elu(lin(x))
                                  + F.selu(lin(x)) + F.hardtanh(lin(x)) + F.logsigmoid(lin(x)) + F.leaky_relu(lin(x), 0.2)
                                  + F.gelu(lin(x), approximate='tanh') + F.relu(lin(x)) + F.softsign(lin(x))
                                  + F.tanhshrink(lin(x))).sum(0),
        'layernorm_module': lambda x: (ln(lin2(torch.tanh(lin(x)))) * lin(x)).sum(-1),
        'einsum': lambda x: torch.einsum('nd,md,nm->n', lin(x), lin(x * 2), ones(N, N)),
        'det_exp': lambda x: torch.linalg.det(lin(x)[:, :5] + eye(5)) * torch.exp(-x.square().sum()),
        'logsumexp_slogdet': lambda x: torch.logsumexp(
            torch.linalg.slogdet(torch.stack([lin(x)[:, :5] + eye(5), lin2(lin(x))[:, :5] + eye(5)]))[1], 0),
        'std_var': lambda x: lin(x).var(dim=-1) + lin(x).std(dim=0).sum() + lin(x).var(dim=-1, unbiased=False),
        'chunk_split_stack': lambda x: torch.cat(torch.chunk(lin(x), 2, dim=-1), 0).sum(0)
        + torch.stack(torch.split(lin(x), 4, dim=-1)).prod(0).sum(0) + torch.split(lin(x), [3, 5], dim=-1)[0].sum(),
        'tril_diag_trace': lambda x: torch.tril(lin(x)[:, :5]).sum(0) + torch.triu(lin(x)[:, :5], 1).sum(0)
        + torch.diagonal(lin(x)[:, :5]) + torch.trace(lin(x)[:, :5]) + torch.diagonal(lin(x), 1).sum(),
        'outer_baddbmm': lambda x: torch.outer(x[:, 0], x[:, 1]).sum(0)
        + torch.baddbmm(ones(1, N, N), x[None], x[None].transpose(1, 2), beta=0.5, alpha=2.0).sum((0, 1)),
        'min_max_clamp': lambda x: torch.minimum(lin(x), lin(x * 2)).sum(0) + lin(x).max(dim=0).values
        + lin(x).clamp(-0.3, 0.3).sum(0) + lin(x).amin(0),
        'powers': lambda x: torch.rsqrt(1 + x.square().sum(-1)) + 1 / (2 + x[:, 0]) + (1 + x.square().sum(-1)) ** 0.3
        + x[:, 1] ** 3,
        'softmax_logsoftmax': lambda x: (F.softmax(lin(x), -1) * F.log_softmax(lin2(lin(x)), -1)).sum(0),
        'masked_fill_where': lambda x: lin(x).masked_fill(torch.eye(N, D) > 0, 0.0).sum(0)
        + torch.where(lin(x) > 0, lin(x), 0.1 * lin(x)).sum(0),
        'cumsum_flip_roll': lambda x: (torch.cumsum(lin(x), 0) * torch.flip(lin(x), [0]) + torch.roll(lin(x), 1, 0)
                                       + torch.roll(lin(x), (1, -2), (0, 1)) + torch.roll(lin(x), 3)).sum(0),
        'gather_index': lambda x: torch.gather(lin(x), 1, _IDX).square().sum(-1) + lin(x)[torch.tensor([0, 2, 2])].sum()
        + torch.gather(lin(x), 0, _IDX.T % N).sum(),
        'solve_inv': lambda x: torch.linalg.solve(lin(x)[:, :5] + 3 * eye(5), x).sum(-1)
        + torch.linalg.inv(lin(x)[:, :5] + 3 * eye(5)).sum(0),
        'expm1_log1p_atan2': lambda x: (torch.expm1(x) + torch.log1p(x.square()) + torch.atan2(x, 1 + x.square())).sum(-1),
        'addcmul_addcdiv': lambda x: torch.addcmul(lin(x), lin(x), lin(x * 2), value=0.5).sum(0)
        + torch.addcdiv(lin(x), lin(x), 2 + lin(x).square()).sum(0),
        'centred_distance': lambda x: (x - x.mean(0, keepdim=True)).pow(2).sum(-1).sqrt(),
        'in_place_updates': _in_place(lin),
        'repeat_tile_pad': lambda x: lin(x).repeat(2, 1).sum(0) + torch.tile(lin(x), (1, 2))[:, :D].sum(0)
        + F.pad(lin(x), (1, 2, 0, 1))[:, 1:D + 1].sum(0) + F.pad(lin(x), (-1, 1), value=0.5).sum(0),
        'embedding': lambda x: (m.emb(torch.tensor([1, 3, 5, 0, 2])) * lin(x)).sum(0),
        'sort_topk_argmax': lambda x: torch.sort(lin(x), dim=-1).values[:, -2:].sum(-1) + torch.topk(lin(x), 2, dim=-1).values.sum(-1)
        + lin(x)[torch.arange(N), lin(x).argmax(-1)] + torch.sort(lin(x), dim=0, descending=True).values[1, :N]
        + torch.gather(lin(x), 1, lin(x * 0.5).argsort(-1))[:, 0],
        'bilinear': lambda x: m.bil(lin(x), lin(x * 0.5)).sum(0),
        'lerp_hypot_logaddexp': lambda x: (torch.lerp(lin(x), lin(x * 2), 0.3) + torch.hypot(lin(x), lin(x * 0.5) + 2)
                                           + torch.logaddexp(lin(x), lin(x * 0.5))).sum(0),
        'norm_dist': lambda x: lin(x).norm() + torch.dist(lin(x), lin(x * 0.5)) + lin(x).norm(dim=-1) + lin(x).norm(p=1)
        + torch.linalg.matrix_norm(lin(x)[:, :5]),
        'xlogy_sigmoid_erf': lambda x: (torch.xlogy(1 + lin(x).square(), 2 + lin(x).square()) + torch.sigmoid(lin(x))
                                        + torch.erf(lin(x))).sum(0),
        'gru_cell': lambda x: m.gru(x, torch.tanh(lin(x))).sum(0),
        'scans': lambda x: (torch.cumprod(1 + 0.1 * lin(x), 0) + torch.cummax(lin(x), 0).values + torch.cummin(lin(x), 1).values
                            + torch.logcumsumexp(lin(x), 0)).sum(0),
        'rounding': lambda x: (torch.sign(lin(x)) * lin(x) + torch.floor(lin(x)).detach() * lin(x) + torch.frac(lin(x))
                               + torch.fmod(lin(x), 0.7) + torch.remainder(lin(x), 0.7)
                               + torch.ceil(lin(x)).detach() * lin(x) + torch.round(lin(x)).detach() * lin(x)).sum(0),
        'full_reductions': lambda x: lin(x).mean() + lin(x).std() + lin(x).var() + lin(x).sum() + lin(x).prod(dim=-1).sum()
        + lin(x).max() + lin(x).min() + lin(x)[0].prod(),
        'shape_juggling': lambda x: torch.bmm(lin(x).reshape(1, N, D), lin(x).reshape(1, N, D).transpose(1, 2).contiguous()).sum((0, 1))
        + lin(x).t().contiguous().flatten()[:N] + sum(torch.unbind(lin(x), 0))[:N] + lin(x).unsqueeze(0).squeeze(0).sum(1)
        + lin(x).movedim(0, 1).sum(0) + lin(x).narrow(0, 1, 2).sum(),
        'gated_and_hard_activations': (
            lambda x: (F.softmin(lin(x), -1) + F.glu(torch.cat([lin(x), lin(x * 0.5)], -1), -1) + F.hardswish(lin(x))
                       + F.hardsigmoid(lin(x)) + F.relu6(lin(x)) + F.softshrink(lin(x), 0.2) + F.hardshrink(lin(x), 0.2)
                       + F.threshold(lin(x), 0.1, 0.0) + F.prelu(lin(x), torch.tensor([0.25], dtype=dt))).sum(0),
            lambda x: (F.softmax(-lin(x), -1) + lin(x) * torch.sigmoid(lin(x * 0.5)) + lin(x) * torch.clamp(lin(x) + 3, 0, 6) / 6
                       + torch.clamp(lin(x) + 3, 0, 6) / 6 + torch.clamp(lin(x), 0, 6)
                       + torch.where(lin(x) > 0.2, lin(x) - 0.2, torch.where(lin(x) < -0.2, lin(x) + 0.2, 0.0 * lin(x)))
                       + torch.where(lin(x).abs() > 0.2, lin(x), 0.0 * lin(x)) + torch.where(lin(x) > 0.1, lin(x), 0.0 * lin(x))
                       + torch.where(lin(x) > 0, lin(x), 0.25 * lin(x))).sum(0)),
        'rrelu_in_evaluation_mode': (lambda x: F.rrelu(lin(x), training=False).sum(0),
                                     lambda x: F.leaky_relu(lin(x), (1 / 8 + 1 / 3) / 2).sum(0)),
        'losses': lambda x: F.mse_loss(lin(x), lin(x * 0.5)) + F.l1_loss(lin(x), lin(x * 0.5)) + F.smooth_l1_loss(lin(x), lin(x * 0.5))
        + F.huber_loss(lin(x), lin(x * 0.5), delta=0.4) + F.cosine_similarity(lin(x), lin(x * 0.5) + 1, dim=-1)
        + F.pairwise_distance(lin(x), lin(x * 0.5)) + F.mse_loss(lin(x), lin(x * 0.5), reduction='sum'),
        'rms_group_norm': lambda x: F.rms_norm(lin(x), (D,)).sum(0) + F.group_norm(lin(x), 2).sum(0)
        + (F.layer_norm(lin(x), (D,)) * lin(x * 0.5)).sum(0),
        'celu_selu': lambda x: (F.celu(lin(x), 0.7) + F.selu(lin(x * 0.5))).sum(0),
        'solve_from_the_right': lambda x: torch.linalg.solve(lin(x)[:, :5] + 3 * eye(5), x.T, left=False).sum(0),
        'tensor_clamp_rounded_division': lambda x: torch.clamp(lin(x), min=lin(x * 0.5) - 0.2, max=lin(x * 0.5) + 0.2).sum(0)
        + (torch.div(lin(x), 0.3, rounding_mode='floor').detach() * lin(x)).sum(0) + lin(x)[0].prod()
        + torch.where(lin(x) > 0, 1.5, lin(x)).sum(0) + torch.where(lin(x) > 0, lin(x), -0.5).sum(0),
    }


def _entry(name):
    def make(dt):
        c = _cases(_M[dt], dt)[name]
        return c if isinstance(c, tuple) else (c, c)

    return make


X = np.random.default_rng(0).normal(size=(2, N, 3)).astype(np.float32)
CONSTRUCTS = {name: _entry(name) for name in _cases(_M[torch.float32], torch.float32)}

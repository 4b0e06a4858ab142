"""CPU stand-ins for ``folx_amd.kernels`` -- TEST INFRASTRUCTURE, used only by the
``not gpu`` tests to exercise the host logic (index algebra, rule composition, masks) in
a container without a GPU.  Each stand-in evaluates the oracle's rule in float64 and
returns float32 torch CPU tensors.  The product never imports this module; without a GPU
and without this patch every rule raises.
"""

import numpy as np
import torch

from oracle import index_algebra as oia
from oracle import rules


def _n(t):
    return t.detach().cpu().numpy().astype(np.float64)


OUT_DTYPE = np.float32  # tests/stagecheck.py asks for float64 references


def _t(a):
    return torch.as_tensor(np.ascontiguousarray(a, dtype=OUT_DTYPE))


def dense(x, jac, lap, W, bias=None, res=None, row_slice=None):
    xs, js, ls = _n(x), _n(jac), _n(lap)
    if row_slice is not None:
        lo, hi = row_slice
        xs, js, ls = xs[..., lo:hi, :], js[..., lo:hi, :], ls[..., lo:hi, :]
    out = rules.dense_rule(xs, js, ls, _n(W), None if bias is None else _n(bias))
    if res is not None:
        out = tuple(o + _n(r) for o, r in zip(out, res))
    return tuple(_t(a) for a in out)


def dense_act(name, x, jac, lap, W, bias=None, param=0.0, res=None):
    z = rules.dense_rule(_n(x), _n(jac), _n(lap), _n(W), None if bias is None else _n(bias))
    nm = {'sigmoid': 'logistic'}.get(name, name)
    out = rules.elementwise_rule(nm, *z, param)
    if res is not None:
        out = tuple(o + _n(r) for o, r in zip(out, res))
    return tuple(_t(a) for a in out)


def dense_act_parts(name, x, lap, jac_parts, widths, broadcast, group, W, bias=None, param=0.0, res=None, pre=None):
    P = jac_parts[0].shape[0]
    lead = tuple(x.shape[:-1])
    R = int(np.prod(lead))
    Js = []
    for J, w, bc in zip(jac_parts, widths, broadcast):
        Jn = _n(J).reshape(P, R // group if bc else R, w)
        Js.append(np.repeat(Jn, group, axis=1) if bc else Jn)
    J = np.concatenate(Js, axis=-1).reshape(P, *lead, sum(widths))
    z = rules.dense_rule(_n(x), J, _n(lap), _n(W), None if bias is None else _n(bias))
    if pre is not None:  # one row per group of consecutive rows, added in front of the activation
        N = z[0].shape[-1]
        rep = lambda t, lead_: np.repeat(_n(t).reshape(*lead_, R // group, N), group, axis=len(lead_)).reshape(*lead_, *lead, N)
        z = (z[0] + rep(pre[0], ()), z[1] + rep(pre[1], (P,)), z[2] + rep(pre[2], ()))
    out = rules.elementwise_rule({'sigmoid': 'logistic'}.get(name, name), *z, param)
    if res is not None:
        out = tuple(o + _n(r) for o, r in zip(out, res))
    return tuple(_t(o) for o in out)


def norm_dense(name, x, jac, lap, gamma, beta, eps, W, bias=None, param=0.0):
    n = layernorm(x, jac, lap, gamma, beta, eps)
    if name is None:
        return dense(*n, W, bias)
    return dense_act(name, *n, W, bias, param)


def dot_two(a, aj, al, b, bj, bl):
    return tuple(_t(t) for t in rules.dot_two_rule(_n(a), _n(aj), _n(al), _n(b), _n(bj), _n(bl)))


def dot_const(a, aj, al, W):
    return tuple(_t(t) for t in rules.dot_const_rule(_n(a), _n(aj), _n(al), _n(W)))


def exp_envelope(d, dj, dl, sigma, pi):
    from oracle import backend as ob

    out = ob.exp_envelope(ob.OArr(_n(d), _n(dj), _n(dl)), _n(sigma), _n(pi))
    return _t(out.x), _t(out.J), _t(out.lap)


def layernorm(x, jac, lap, gamma, beta, eps):
    from oracle import backend as ob

    out = ob.layer_norm(ob.OArr(_n(x), _n(jac), _n(lap)), None if gamma is None else _n(gamma),
                        None if beta is None else _n(beta), eps)
    return _t(out.x), _t(out.J), _t(out.lap)


def elementwise(name, x, jac, lap, param=0.0, inplace=False):
    nm = {'sigmoid': 'logistic'}.get(name, name)
    return tuple(_t(a) for a in rules.elementwise_rule(nm, _n(x), _n(jac), _n(lap), param))


def binary(op, a, aj, al, b, bj, bl):
    rule = {'mul': rules.mul_rule, 'div': rules.div_rule, 'add': rules.add_rule,
            'sub': lambda *t: rules.add_rule(*t, sign=-1.0),
            'min': lambda *t: rules.minmax_rule(*t, is_max=False),
            'max': lambda *t: rules.minmax_rule(*t, is_max=True)}[op]
    A = [_n(t) for t in (a, aj, al)]
    Bb = [_n(t) for t in (b, bj, bl)]
    shp = np.broadcast_shapes(A[0].shape, Bb[0].shape)
    P = A[1].shape[0]
    A = [np.broadcast_to(A[0], shp), np.broadcast_to(A[1], (P, *shp)), np.broadcast_to(A[2], shp)]
    Bb = [np.broadcast_to(Bb[0], shp), np.broadcast_to(Bb[1], (P, *shp)), np.broadcast_to(Bb[2], shp)]
    return tuple(_t(t) for t in rule(*A, *Bb))


def mul_sparse(a, aj, al, b, bj, bl, index):
    ix = index.cpu().numpy()
    bjn = _n(bj)
    P = aj.shape[0]
    dense = np.zeros((P, *bjn.shape[1:]))
    flat = dense.reshape(P, bjn.shape[1], -1)
    src = bjn.reshape(bjn.shape[0], bjn.shape[1], -1)
    for s in range(ix.shape[0]):
        for e in range(ix.shape[1]):
            if ix[s, e] >= 0:
                flat[ix[s, e], :, e] += src[s, :, e]
    return tuple(_t(t) for t in rules.mul_rule(_n(a), _n(aj), _n(al), _n(b), dense, _n(bl)))


def rows_affine(inp, rows, row_shape, out_shape, c=None, d=None, alpha=1.0, beta=1.0):
    a = _n(inp).reshape(rows, *row_shape)
    nd = len(out_shape)
    a = a.reshape(rows, *([1] * (nd - len(row_shape))), *row_shape)
    out = alpha * np.broadcast_to(a, (rows, *out_shape))
    if c is not None:
        out = out * _n(c)
    if d is not None:
        out = out + beta * _n(d)
    return _t(np.broadcast_to(out, (rows, *out_shape)))


def reduce_sum(inp, rows, outer, red, inner, alpha=1.0, window=None):
    v = _n(inp).reshape(rows, outer, red, inner)
    if window is not None:
        v = v[:, :, window[0]:window[1]]
    return _t(alpha * v.sum(2))


def reduce_max(inp, outer, red, inner):
    return _t(_n(inp).reshape(outer, red, inner).max(1))


def gather_rows(data, take, k_out, n_slots, B, S_outer, S_inner):
    d = _n(data).reshape(data.shape[0], B, S_outer, S_inner)
    tk = take.cpu().numpy().reshape(k_out, n_slots, S_outer)
    out = np.zeros((k_out, B, S_outer, S_inner))
    for t in range(k_out):
        for s in range(n_slots):
            for so in range(S_outer):
                r = tk[t, s, so]
                if r >= 0:
                    out[t, :, so] += d[r, :, so]
    return _t(out.reshape(k_out, B, S_outer * S_inner))


def gather_reduce_rows(data, take, k_out, n_slots, B, O, RED, IV, IC, alpha=1.0):
    d = _n(data).reshape(data.shape[0], B, O, RED, IV, IC)
    tk = take.cpu().numpy().reshape(k_out, n_slots, O, IV)
    out = np.zeros((k_out, B, O, IV, IC))
    for t in range(k_out):
        for s_ in range(n_slots):
            for o in range(O):
                for iv in range(IV):
                    e = tk[t, s_, o, iv]
                    if e >= 0:
                        out[t, :, o, iv] += d[e // RED, :, o, e % RED, iv]
    return _t(alpha * out.reshape(k_out, B, O * IV * IC))


def scatter_add_rows(data, idx, k_out, B, S_outer, S_inner, out=None):
    d = _n(data).reshape(data.shape[0], B, S_outer, S_inner)
    ix = idx.cpu().numpy()
    acc = np.zeros((k_out, B, S_outer, S_inner)) if out is None else _n(out).reshape(k_out, B, S_outer, S_inner).copy()
    for r in range(d.shape[0]):
        for so in range(S_outer):
            if ix[r, so] >= 0:
                acc[ix[r, so], :, so] += d[r, :, so]
    res = _t(acc.reshape(k_out, B, S_outer * S_inner))
    if out is not None:
        if OUT_DTYPE != np.float32:  # a float64 reference evaluation never writes into its arguments
            return res.reshape(out.shape)
        out.reshape(k_out, B, S_outer * S_inner).copy_(res)
        return out
    return res


def gather_cols(data, table, S_inner=1):
    d = _n(data)
    t = table.cpu().numpy()
    RB = d.shape[0]
    d = d.reshape(RB, -1, S_inner)
    out = np.zeros((RB, t.shape[0], S_inner))
    for s in range(t.shape[1]):
        valid = t[:, s] >= 0
        out[:, valid] += d[:, t[valid, s]]
    return _t(out.reshape(RB, -1))


def slogdet(A, AJ, AL, row_axis=None, factor=None):
    a, aj, al = _n(A), _n(AJ), _n(AL)
    if factor is not None:
        F, FJ, FL, index = factor
        ix, fj = index.cpu().numpy(), _n(FJ)
        dense = np.zeros_like(aj).reshape(aj.shape[0], aj.shape[1], -1)
        src = fj.reshape(fj.shape[0], fj.shape[1], -1)
        for s_ in range(ix.shape[0]):
            for e in range(ix.shape[1]):
                if ix[s_, e] >= 0:
                    dense[ix[s_, e], :, e] += src[s_, :, e]
        a, aj, al = rules.mul_rule(a, aj, al, _n(F), dense.reshape(aj.shape), _n(FL))
    if row_axis is not None:
        ra = row_axis % a.ndim
        a, al = np.moveaxis(a, ra, -2), np.moveaxis(al, ra, -2)
        aj = np.moveaxis(aj, ra + 1, -2)
    sign, (ld, jac, lap) = rules.slogdet_rule(a, aj, al)
    return _t(sign), _t(ld), _t(jac), _t(lap)


def sparse_slogdet(A, AJ, AL, take, cols, rows, transposed):
    take, cols, rows = (t.cpu().numpy().astype(np.int64) for t in (take, cols, rows))
    a, aj, al = _n(A), _n(AJ), _n(AL)
    k, n = aj.shape[0], a.shape[-1]
    if transposed:
        # the tables describe A^T and address A_jac as stored: run the oracle on A^T
        t, rem = np.divmod(np.where(take >= 0, take, 0), n * n)
        r, c = np.divmod(rem, n)
        take = np.where(take >= 0, (t * n + c) * n + r, -1)
        a, aj, al = (np.swapaxes(v, -1, -2) for v in (a, aj, al))
    take = np.where(take >= 0, take, k * n * n)
    sign, (ld, jac, lap) = rules.sparse_slogdet_rule(
        a, aj, al, dict(take=take, cols=cols, rows=rows, per_entry=False))
    return _t(sign), _t(ld), _t(jac), _t(lap)


def slogdet_any(A, AJ, AL):
    return slogdet(A, AJ, AL)


def inv_any(A, AJ, AL):
    return inv(A, AJ, AL)


def inv(A, AJ, AL):
    return tuple(_t(v) for v in rules.inv_rule(_n(A), _n(AJ), _n(AL)))


def solve(A, AJ, AL, b, bJ, bL, P):
    opt = lambda v: None if v is None else _n(v)
    return tuple(_t(v) for v in rules.solve_rule(_n(A), opt(AJ), opt(AL), _n(b), opt(bJ), opt(bL)))


def mhsa(q, qj, ql, k, kj, kl, v, vj, vl, mask=None, input_mask=None, edge=None):
    m = None if mask is None else mask.cpu().numpy().astype(bool)
    im = None if input_mask is None else input_mask.cpu().numpy().astype(bool)
    ed = () if edge is None else tuple(_n(t) for t in edge)
    return tuple(_t(a) for a in rules.mhsa_rule(*[_n(t) for t in (q, qj, ql, k, kj, kl, v, vj, vl)], m, im, *ed))


def mhsa_sparse(q, qs, ql, k, ks, kl, v, vs, vl, index, P, all_rows_named):
    ix = index.cpu().numpy()

    def dense(xs):
        xs = _n(xs)
        J = np.zeros((P, *xs.shape[1:]))
        for s in range(ix.shape[0]):
            for e in range(ix.shape[1]):
                if ix[s, e] >= 0:
                    J[ix[s, e], :, e] = xs[s, :, e]
        return J

    return tuple(_t(a) for a in rules.mhsa_rule(_n(q), dense(qs), _n(ql), _n(k), dense(ks), _n(kl),
                                                _n(v), dense(vs), _n(vl)))


KERNEL_NAMES = ('dense', 'dense_act', 'dense_act_parts', 'norm_dense', 'dot_two', 'dot_const', 'exp_envelope', 'layernorm', 'elementwise', 'binary',
                'mul_sparse', 'rows_affine', 'reduce_sum', 'reduce_max', 'gather_rows', 'gather_reduce_rows', 'gather_cols', 'scatter_add_rows',
                'slogdet', 'sparse_slogdet', 'slogdet_any', 'inv', 'inv_any', 'solve', 'mhsa', 'mhsa_sparse')


def install(monkeypatch):
    import folx_amd.interpreter as interp
    import folx_amd.kernels as K

    for name in KERNEL_NAMES:
        monkeypatch.setattr(K, name, globals()[name])
    monkeypatch.setattr(interp, '_device', lambda: torch.device('cpu'))

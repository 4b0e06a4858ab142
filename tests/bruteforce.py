"""Brute-force fp64 oracle: value, Jacobian and trace of the Hessian by torch autograd.

Same method as the reference's own test base class (test/laplacian_testcase.py:22-49:
Jacobian by AD, Laplacian as the trace of the full AD Hessian in float64).  A model
written against the operator namespace runs here on plain fp64 torch tensors of ONE
walker; ``brute_force`` loops over walkers.
"""

import math

import numpy as np
import torch


class plain:
    """Operator namespace on plain torch tensors (single walker, no derivatives)."""

    float64 = torch.float64

    @staticmethod
    def _c(c, like):
        if isinstance(c, torch.Tensor):
            return c.to(like.dtype)
        return torch.as_tensor(np.asarray(c), dtype=like.dtype)

    @staticmethod
    def dot(h, W, b=None, residual=None, row_slice=None, act=None, norm=None):
        if norm is not None:
            h = plain.layer_norm(h, *norm)
        if row_slice is not None:
            h = h[..., row_slice[0]:row_slice[1], :]
        y = h @ plain._c(W, h)
        y = y if b is None else y + plain._c(b, h)
        if act is not None:
            y = getattr(plain, {'logistic': 'sigmoid'}.get(act, act))(y)
        return y if residual is None else residual + y

    @staticmethod
    def exp_envelope(d, sigma, pi):
        return (torch.exp(-d[..., None] * plain._c(sigma, d)) * plain._c(pi, d)).sum(-2)

    @staticmethod
    def layer_norm(h, gamma=None, beta=None, eps=1e-5, lazy=False):
        mu = h.mean(-1, keepdim=True)
        c = h - mu
        y = c * torch.rsqrt((c * c).mean(-1, keepdim=True) + eps)
        if gamma is not None:
            y = y * plain._c(gamma, h)
        return y if beta is None else y + plain._c(beta, h)

    tanh = staticmethod(torch.tanh)
    exp = staticmethod(torch.exp)
    log = staticmethod(torch.log)
    sqrt = staticmethod(torch.sqrt)
    rsqrt = staticmethod(torch.rsqrt)
    square = staticmethod(torch.square)
    sigmoid = staticmethod(torch.sigmoid)
    logistic = staticmethod(torch.sigmoid)
    softplus = staticmethod(torch.nn.functional.softplus)
    silu = staticmethod(torch.nn.functional.silu)
    sin = staticmethod(torch.sin)
    cos = staticmethod(torch.cos)
    abs = staticmethod(torch.abs)
    negative = staticmethod(torch.neg)
    log1p = staticmethod(torch.log1p)
    reciprocal = staticmethod(torch.reciprocal)
    expm1 = staticmethod(torch.expm1)
    sinh, cosh, tan = staticmethod(torch.sinh), staticmethod(torch.cosh), staticmethod(torch.tan)
    arcsin, arccos, arctan = staticmethod(torch.asin), staticmethod(torch.acos), staticmethod(torch.atan)
    arcsinh, arccosh, arctanh = staticmethod(torch.asinh), staticmethod(torch.acosh), staticmethod(torch.atanh)
    erf, erfc, erf_inv = staticmethod(torch.erf), staticmethod(torch.erfc), staticmethod(torch.erfinv)
    cbrt = staticmethod(lambda t: torch.sign(t) * torch.abs(t) ** (1.0 / 3.0))
    lgamma = staticmethod(torch.lgamma)
    digamma = staticmethod(torch.digamma)

    @staticmethod
    def power(a, c):
        if torch.is_tensor(c) or not np.isscalar(c):
            return (a if torch.is_tensor(a) else plain._c(a, c)) ** (c if torch.is_tensor(c) else plain._c(c, a))
        return a ** float(c)

    @staticmethod
    def integer_pow(a, n):
        return a**n

    @staticmethod
    def _b(a, b):
        if isinstance(a, torch.Tensor) and not isinstance(b, torch.Tensor):
            b = plain._c(b, a)
        elif isinstance(b, torch.Tensor) and not isinstance(a, torch.Tensor):
            a = plain._c(a, b)
        return a, b

    @staticmethod
    def add(a, b):
        a, b = plain._b(a, b)
        return a + b

    @staticmethod
    def subtract(a, b):
        a, b = plain._b(a, b)
        return a - b

    @staticmethod
    def multiply(a, b):
        a, b = plain._b(a, b)
        return a * b

    @staticmethod
    def divide(a, b):
        a, b = plain._b(a, b)
        return a / b

    @staticmethod
    def sum(a, axis=None, keepdims=False, window=None):
        if axis is None:
            return a.sum()
        if window is not None:
            a = a.narrow(axis, window[0], window[1] - window[0])
        return a.sum(dim=axis, keepdim=keepdims)

    @staticmethod
    def mean(a, axis=None, keepdims=False, window=None):
        if axis is None:
            return a.mean()
        if window is not None:
            a = a.narrow(axis, window[0], window[1] - window[0])
        return a.mean(dim=axis, keepdim=keepdims)

    @staticmethod
    def reshape(a, shape):
        return a.reshape(tuple(shape))

    @staticmethod
    def transpose(a, axes):
        return a.permute(tuple(axes))

    @staticmethod
    def swapaxes(a, i, j):
        return a.transpose(i, j)

    @staticmethod
    def expand_dims(a, axis):
        return a.unsqueeze(axis)

    @staticmethod
    def broadcast_to(a, shape, lazy=False):
        return a.expand(tuple(shape))

    @staticmethod
    def getitem(a, idx):
        return a[idx]

    @staticmethod
    def concatenate(arrs, axis=-1, lazy=False):
        like = [t for t in arrs if isinstance(t, torch.Tensor)][0]
        return torch.cat([plain._c(t, like) for t in arrs], dim=axis)

    @staticmethod
    def stop_gradient(a):
        return a.detach()

    @staticmethod
    def amax_const(a, axis, keepdims=False):
        return a.detach().amax(dim=axis, keepdim=keepdims)

    @staticmethod
    def matmul(a, b):
        a, b = plain._b(a, b)
        return a @ b

    @staticmethod
    def einsum(subscripts, *ops):
        like = [o for o in ops if torch.is_tensor(o)][0]
        return torch.einsum(subscripts, *[o if torch.is_tensor(o) else plain._c(o, like) for o in ops])

    @staticmethod
    def dot_general(lhs, rhs, dimension_numbers):
        """jax.lax.dot_general: output axes are batch, lhs free, rhs free."""
        a, b = plain._b(lhs, rhs)
        (lc, rc), (lb, rb) = dimension_numbers
        lc, lb = [i % a.ndim for i in lc], [i % a.ndim for i in lb]
        rc, rb = [i % b.ndim for i in rc], [i % b.ndim for i in rb]
        lf = [i for i in range(a.ndim) if i not in lc + lb]
        rf = [i for i in range(b.ndim) if i not in rc + rb]
        at = a.permute(*lb, *lf, *lc)
        bt = b.permute(*rb, *rc, *rf)
        bs = [a.shape[i] for i in lb]
        y = at.reshape(*bs, int(np.prod([a.shape[i] for i in lf])), -1) @ bt.reshape(
            *bs, -1, int(np.prod([b.shape[i] for i in rf])))
        return y.reshape(*bs, *[a.shape[i] for i in lf], *[b.shape[i] for i in rf])

    @staticmethod
    def softmax(a, axis=-1):
        return torch.softmax(a, dim=axis)

    @staticmethod
    def det(A):
        n = A.shape[-1]
        if n == 1:
            return A[..., 0, 0]
        # Laplace expansion along the first row: pure arithmetic, safe under any AD mode
        out = 0
        for j in range(n):
            minor = torch.cat([A[..., 1:, :j], A[..., 1:, j + 1:]], dim=-1)
            out = out + ((-1) ** j) * A[..., 0, j] * plain.det(minor)
        return out

    @staticmethod
    def inv(A):
        # adjugate / determinant by cofactor expansion: pure arithmetic under any AD mode
        n = A.shape[-1]
        if n == 1:
            return 1.0 / A
        rows = []
        for i in range(n):
            cols = []
            for j in range(n):
                # entry (i, j) of the inverse = cofactor (j, i) / det
                minor = torch.cat([A[..., :j, :], A[..., j + 1:, :]], dim=-2)
                minor = torch.cat([minor[..., :, :i], minor[..., :, i + 1:]], dim=-1)
                cols.append(((-1) ** (i + j)) * plain.det(minor))
            rows.append(torch.stack(cols, dim=-1))
        return torch.stack(rows, dim=-2) / plain.det(A)[..., None, None]

    @staticmethod
    def solve(A, b):
        A, b = plain._b(A, b)
        if b.ndim == 1:
            return (plain.inv(A) @ b[..., None])[..., 0]
        return plain.inv(A) @ b

    @staticmethod
    def minimum(a, b):
        a, b = plain._b(a, b)
        return torch.minimum(a, b)

    @staticmethod
    def maximum(a, b):
        a, b = plain._b(a, b)
        return torch.maximum(a, b)

    @staticmethod
    def scatter(operand, idx, updates, mode='set'):
        # one scalar at a time, so that every AD mode sees plain arithmetic
        like = operand if isinstance(operand, torch.Tensor) else updates
        operand = plain._c(operand, like)
        shape = tuple(operand.shape)
        tpos = np.arange(operand.numel()).reshape(shape)[idx]
        upd = plain._c(updates, like).expand(tpos.shape).reshape(-1)
        flat = [v for v in operand.reshape(-1)]
        for e, p in enumerate(tpos.reshape(-1)):
            if mode == 'set':
                flat[p] = upd[e]
            elif mode == 'add':
                flat[p] = flat[p] + upd[e]
            elif mode == 'min':
                flat[p] = torch.minimum(flat[p], upd[e])
            else:
                flat[p] = torch.maximum(flat[p], upd[e])
        return torch.stack(flat).reshape(shape)

    @staticmethod
    def clip(a, lo=None, hi=None):
        return torch.clamp(a, lo, hi)

    @staticmethod
    def where(cond, a, b):
        c = cond.bool() if isinstance(cond, torch.Tensor) else torch.as_tensor(np.asarray(cond)).bool()
        a, b = plain._b(a, b)
        return torch.where(c, a, b)

    @staticmethod
    def cumsum(a, axis=-1):
        return torch.cumsum(a, dim=axis)

    @staticmethod
    def amax(a, axis=-1):
        return a.amax(dim=axis)

    @staticmethod
    def amin(a, axis=-1):
        return a.amin(dim=axis)

    @staticmethod
    def prod(a, axis=-1):
        return a.prod(dim=axis)

    @staticmethod
    def flip(a, axis):
        return torch.flip(a, [axis] if np.isscalar(axis) else list(axis))

    @staticmethod
    def pad(a, pad_width, constant_values=0.0):
        pw = [tuple(p) for p in pad_width] if np.ndim(pad_width) == 2 else [tuple(pad_width)] * a.ndim
        flat = [v for p in reversed(pw) for v in p]
        return torch.nn.functional.pad(a, flat, value=constant_values)

    @staticmethod
    def lax_pad(a, padding_value, padding_config):
        """jax.lax.pad element by element: output position q of an axis holds operand entry j when
        q = low + j (interior + 1), the padding value otherwise."""
        cfg = [tuple(int(v) for v in c) for c in padding_config]
        sizes = [max(lo + n + max(n - 1, 0) * it + hi, 0) for n, (lo, hi, it) in zip(a.shape, cfg)]
        pv = padding_value if torch.is_tensor(padding_value) else torch.tensor(float(padding_value), dtype=a.dtype)
        out = []
        for q in np.ndindex(*sizes):
            src = []
            for qa, n, (lo, hi, it) in zip(q, a.shape, cfg):
                j, r = divmod(qa - lo, it + 1)
                src.append(j if r == 0 and 0 <= j < n else None)
            out.append(pv.reshape(()) if any(v is None for v in src) else a[tuple(src)])
        return torch.stack(out).reshape(sizes)

    relu = staticmethod(torch.relu)
    leaky_relu = staticmethod(lambda a, negative_slope=0.01: torch.nn.functional.leaky_relu(a, negative_slope))
    elu = staticmethod(lambda a, alpha=1.0: torch.nn.functional.elu(a, alpha))
    gelu = staticmethod(lambda a, approximate=True: torch.nn.functional.gelu(a, approximate='tanh' if approximate else 'none'))
    log_softmax = staticmethod(lambda a, axis=-1: torch.log_softmax(a, dim=axis))
    var = staticmethod(lambda a, axis=None, keepdims=False: torch.var(a, dim=axis, unbiased=False, keepdim=keepdims))
    std = staticmethod(lambda a, axis=None, keepdims=False: torch.std(a, dim=axis, unbiased=False, keepdim=keepdims))
    norm = staticmethod(lambda a, axis=None, keepdims=False: torch.linalg.vector_norm(a, dim=axis, keepdim=keepdims))
    vdot = staticmethod(lambda a, b: torch.dot(plain._c(a, b).reshape(-1) if not torch.is_tensor(a) else a.reshape(-1),
                                               plain._c(b, a).reshape(-1) if not torch.is_tensor(b) else b.reshape(-1)))
    tensordot = staticmethod(lambda a, b, axes=2: torch.tensordot(
        a if torch.is_tensor(a) else plain._c(a, b), b if torch.is_tensor(b) else plain._c(b, a),
        dims=axes if isinstance(axes, int) else [list((v,) if isinstance(v, int) else v) for v in axes]))
    inner = staticmethod(lambda a, b: torch.inner(a if torch.is_tensor(a) else plain._c(a, b), b if torch.is_tensor(b) else plain._c(b, a)))
    outer = staticmethod(lambda a, b: torch.outer(a.reshape(-1), b.reshape(-1)))
    moveaxis = staticmethod(torch.movedim)
    take = staticmethod(lambda a, indices, axis=None: torch.take(a, torch.as_tensor(np.asarray(indices))) if axis is None
                        else torch.index_select(a, axis, torch.as_tensor(np.asarray(indices)).reshape(-1)).reshape(
                            *a.shape[:axis % a.ndim], *np.shape(indices), *a.shape[axis % a.ndim + 1:]))
    diagonal = staticmethod(lambda a, offset=0: torch.diagonal(a, offset, -2, -1))
    trace = staticmethod(lambda a, offset=0: torch.diagonal(a, offset, -2, -1).sum(-1))
    roll = staticmethod(lambda a, shift, axis: torch.roll(a, shift, axis))
    repeat = staticmethod(lambda a, repeats, axis: torch.repeat_interleave(a, repeats, dim=axis))

    arctan2 = staticmethod(lambda y, x: torch.atan2(y if torch.is_tensor(y) else plain._c(y, x), plain._c(x, y) if torch.is_tensor(y) else x))
    remainder = staticmethod(lambda a, b: torch.fmod(a, plain._c(b, a)))
    fmod = remainder
    exp2 = staticmethod(torch.exp2)
    split = staticmethod(lambda a, k, axis=0: list(torch.split(a, a.shape[axis] // k, dim=axis)) if np.isscalar(k)
                         else list(torch.tensor_split(a, list(k), dim=axis)))
    stack = staticmethod(lambda arrs, axis=0: torch.stack(list(arrs), dim=axis))
    tile = staticmethod(lambda a, reps: torch.tile(a, (reps,) if np.isscalar(reps) else tuple(reps)))
    trunc = staticmethod(lambda a: torch.trunc(a).detach())

    @staticmethod
    def dynamic_slice(a, start, sizes):
        idx = tuple(slice(int(np.clip(s0, 0, n - sz)), int(np.clip(s0, 0, n - sz)) + sz)
                    for s0, sz, n in zip(start, sizes, a.shape))
        return a[idx]

    @staticmethod
    def dynamic_update_slice(a, u, start):
        idx = tuple(slice(int(np.clip(s0, 0, n - un)), int(np.clip(s0, 0, n - un)) + un)
                    for s0, un, n in zip(start, u.shape, a.shape))
        out = a.clone()
        out[idx] = u
        return out

    greater = staticmethod(lambda a, b: (a > plain._c(b, a)).detach())
    less = staticmethod(lambda a, b: (a < plain._c(b, a)).detach())
    floor = staticmethod(lambda a: torch.floor(a).detach())
    logaddexp = staticmethod(torch.logaddexp)

    @staticmethod
    def cumprod(a, axis=-1):
        return torch.cumprod(a, dim=axis)

    @staticmethod
    def cummax(a, axis=-1):
        return torch.cummax(a, dim=axis).values

    @staticmethod
    def cummin(a, axis=-1):
        return torch.cummin(a, dim=axis).values

    @staticmethod
    def sign(a):
        return torch.sign(a.detach())

    @staticmethod
    def squeeze(a, axis):
        return a.squeeze(axis)

    @staticmethod
    def logsumexp(a, axis=-1, b=None):
        m = a.detach().amax(dim=axis, keepdim=True)
        e = torch.exp(a - m)
        if b is not None:
            e = e * plain._c(b, a)
        s = e.sum(dim=axis)
        return torch.log(torch.abs(s)) + m.reshape(s.shape), torch.sign(s.detach())

    @staticmethod
    def slogdet(A, row_axis=None, factor=None):
        if factor is not None:
            A = A * factor
        if row_axis is not None:
            A = torch.movedim(A, row_axis, -2)
        sign, ld = torch.linalg.slogdet(A)
        return sign.detach(), ld

    @staticmethod
    def multi_head_self_attention(q, k, v, mask=None, input_mask=None, bias=None):
        # q, k, v: (n, H, d); softmax(q k^T (+ bias)) v, no 1/sqrt(d) inside
        s = torch.einsum('ihd,jhd->ihj', q, k)
        if bias is not None:
            s = s + bias
        if mask is not None:
            m = torch.as_tensor(np.asarray(mask), dtype=torch.bool)
            sq = m[:, None, None] & m[None, None, :]
            s = torch.where(sq, s, torch.full_like(s, -1e40))
        p = torch.softmax(s, dim=-1)
        return torch.einsum('ihj,jhd->ihd', p, v)


def brute_force_single(fn, x):
    """fn: tensor (s) -> tensor (out).  Returns (y, J (n_in, *out), lap (*out)) in fp64."""
    x = torch.as_tensor(np.asarray(x), dtype=torch.float64)
    flat = x.reshape(-1)

    def f(z):
        return fn(z.reshape(x.shape))

    y = f(flat)
    J = torch.func.jacrev(f)(flat)  # (*out, n)
    # forward-over-reverse: torch's forward-over-forward through linalg.det / slogdet
    # returns wrong second derivatives (checked against an explicit cofactor expansion in
    # tests/test_oracle_rules.py), so the Hessian is never taken that way here.
    H = torch.func.jacfwd(torch.func.jacrev(f))(flat)  # (*out, n, n)
    lap = torch.diagonal(H, dim1=-2, dim2=-1).sum(-1)
    J = torch.movedim(J, -1, 0)
    return y.detach().numpy(), J.detach().numpy(), lap.detach().numpy()


def brute_force(fn, x):
    """x: (B, *s) numpy.  Returns x (B, *out), J (n_in, B, *out), lap (B, *out)."""
    ys, Js, Ls = [], [], []
    for b in range(x.shape[0]):
        y, J, L = brute_force_single(fn, x[b])
        ys.append(y), Js.append(J), Ls.append(L)
    return np.stack(ys, 0), np.stack(Js, 1), np.stack(Ls, 0)

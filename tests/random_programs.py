"""Seeded random compositions of the rules: a program is a short list of steps over a pool of values that all
derive from one input vector; the same program runs on the oracle backend, on the product and (for the
oracle's own pin) on torch under AD.  What this exercises is the host side of the path -- mask propagation
through indexing, merges of sparse Jacobians in binary rules, reductions over sparse axes, the dense switch
(folx/jvp.py:273-413, folx/api.py:230-249, folx/utils.py:499-588) -- in combinations nobody wrote by hand."""

import numpy as np

N_IN = 12
_SHAPES = [(12,), (3, 4), (4, 3), (2, 6), (6, 2), (2, 3, 2), (2, 2, 3), (3, 2, 2)]
_UNARY = ['sin', 'cos', 'tanh', 'square', 'sigmoid']
_BINARY = ['add', 'subtract', 'multiply', 'divide']
_MORE = ['inv_spd', 'solve_spd', 'attention', 'scatter', 'cumprod', 'cummax', 'prod', 'amin', 'minimum', 'maximum', 'clip',
         'layer_norm', 'where_data', 'abs_sqrt']


def _factorizations(n):
    out = [(n,)]
    for a in range(2, n):
        if n % a == 0:
            out.append((a, n // a))
            for b in range(2, n // a):
                if (n // a) % b == 0:
                    out.append((a, b, n // a // b))
    return out


def generate(seed: int, n_steps: int = 7, n_in: int = N_IN, more: bool = False):
    """Returns a list of steps ``(op, operand indices, static arguments)``; shapes are tracked while drawing
    so that every step is valid.  Value 0 is the input (``n_in`` entries), value 1 the input reshaped.  ``more``: also
    the second family of steps (inverse / solve, attention, scatter, scans, min / max, clip, LayerNorm, a ``where`` whose
    condition depends on the data)."""
    rng = np.random.default_rng(seed)
    first_shapes = _SHAPES if n_in == N_IN else _factorizations(n_in)
    first = first_shapes[rng.integers(len(first_shapes))]
    steps = [('reshape', (0,), (first,))]
    shapes = [(n_in,), first]          # value 0: the raw input; value 1: reshaped
    for _ in range(n_steps):
        for _attempt in range(20):
            i = int(rng.integers(1, len(shapes)))
            s = shapes[i]
            kind = rng.choice(['unary', 'binary', 'reshape', 'transpose', 'slice', 'sum', 'dot', 'concat', 'broadcast',
                               'flip', 'where', 'cumsum', 'amax', 'take', 'binary_const', 'mean_keep', 'pad',
                               'matmul_t', 'softmax', 'logsumexp', 'logdet_spd'] + (_MORE if more else []))
            size = int(np.prod(s, dtype=int))
            if kind == 'unary':
                steps.append((str(rng.choice(_UNARY)), (i,), ())); shapes.append(s)
            elif kind == 'binary':
                # a partner of the same shape, or one that broadcasts (a trailing-axes suffix, or size-1 axes)
                cands = [j for j in range(1, len(shapes)) if shapes[j] == s or
                         (len(shapes[j]) <= len(s) and shapes[j] == s[len(s) - len(shapes[j]):]) or
                         (len(shapes[j]) == len(s) and all(a == b or a == 1 for a, b in zip(shapes[j], s)))]
                if not cands:
                    continue
                j = int(rng.choice(cands))
                op = str(rng.choice(_BINARY))
                steps.append((op, (i, j) if rng.random() < 0.5 else (j, i), ())); shapes.append(s)
            elif kind == 'binary_const':
                c = rng.normal(size=s[-1:] if rng.random() < 0.5 else ()).astype(np.float32)
                steps.append((str(rng.choice(['add', 'multiply'])), (i,), (c,))); shapes.append(s)
            elif kind == 'reshape':
                if size < 2:
                    continue
                f = _factorizations(size)
                t = f[rng.integers(len(f))]
                steps.append(('reshape', (i,), (t,))); shapes.append(tuple(t))
            elif kind == 'transpose':
                if len(s) < 2:
                    continue
                perm = tuple(int(p) for p in rng.permutation(len(s)))
                steps.append(('transpose', (i,), (perm,))); shapes.append(tuple(s[p] for p in perm))
            elif kind == 'slice':
                if not s:
                    continue
                ax = int(rng.integers(len(s)))
                if s[ax] < 2:
                    continue
                lo = int(rng.integers(0, s[ax] - 1))
                hi = int(rng.integers(lo + 1, s[ax] + 1))
                st = int(rng.choice([1, 1, 2]))
                idx = tuple(slice(lo, hi, st) if a == ax else slice(None) for a in range(ax + 1))
                n = len(range(lo, hi, st))
                steps.append(('getitem', (i,), (idx,))); shapes.append((*s[:ax], n, *s[ax + 1:]))
            elif kind in ('sum', 'mean_keep'):
                if not s:
                    continue
                ax = int(rng.integers(len(s)))
                keep = kind == 'mean_keep'
                steps.append(('mean' if keep else 'sum', (i,), (ax, keep)))
                shapes.append((*s[:ax], 1, *s[ax + 1:]) if keep else (*s[:ax], *s[ax + 1:]))
            elif kind == 'dot':
                if not s:
                    continue
                n_out = int(rng.integers(1, 5))
                W = (rng.normal(size=(s[-1], n_out)) / np.sqrt(s[-1])).astype(np.float32)
                steps.append(('dot', (i,), (W,))); shapes.append((*s[:-1], n_out))
            elif kind == 'concat':
                if not s:
                    continue
                ax = int(rng.integers(len(s)))
                cands = [j for j in range(1, len(shapes)) if len(shapes[j]) == len(s) and
                         all(a == b for k, (a, b) in enumerate(zip(shapes[j], s)) if k != ax)]
                j = int(rng.choice(cands))
                steps.append(('concatenate', (i, j), (ax,)))
                shapes.append((*s[:ax], s[ax] + shapes[j][ax], *s[ax + 1:]))
            elif kind == 'broadcast':
                if len(s) >= 3 or size > 24:
                    continue
                lead = int(rng.integers(2, 4))
                steps.append(('broadcast_to', (i,), ((lead, *s),))); shapes.append((lead, *s))
            elif kind == 'flip':
                if not s:
                    continue
                steps.append(('flip', (i,), (int(rng.integers(len(s))),))); shapes.append(s)
            elif kind == 'where':
                m = rng.random(size=s) < 0.5
                cands = [j for j in range(1, len(shapes)) if shapes[j] == s]
                j = int(rng.choice(cands))
                steps.append(('where', (i, j), (m,))); shapes.append(s)
            elif kind == 'cumsum':
                if not s:
                    continue
                steps.append(('cumsum', (i,), (int(rng.integers(len(s))),))); shapes.append(s)
            elif kind == 'amax':
                if not s or s[-1] < 2:
                    continue
                steps.append(('amax', (i,), (len(s) - 1,))); shapes.append(s[:-1])
            elif kind == 'take':
                if not s:
                    continue
                ax = int(rng.integers(len(s)))
                idx = rng.integers(0, s[ax], size=int(rng.integers(1, 5)))
                steps.append(('take', (i,), (idx, ax))); shapes.append((*s[:ax], len(idx), *s[ax + 1:]))
            elif kind == 'pad':
                if not s or size > 36:
                    continue
                cfg = tuple((int(rng.integers(-1, 2)) if n > 2 else int(rng.integers(0, 2)), int(rng.integers(0, 2)),
                             int(rng.integers(0, 2))) for n in s)
                out = tuple(max(lo + n + max(n - 1, 0) * it + hi, 0) for n, (lo, hi, it) in zip(s, cfg))
                if min(out) < 1:
                    continue
                steps.append(('lax_pad', (i,), (float(rng.normal()), cfg))); shapes.append(out)
            elif kind == 'matmul_t':
                # product of two derivative-carrying operands: v (..., m, k) times the transposed partner (..., k, m)
                if len(s) < 2:
                    continue
                cands = [j for j in range(1, len(shapes)) if shapes[j] == s]
                j = int(rng.choice(cands))
                steps.append(('matmul_t', (i, j), ())); shapes.append((*s[:-1], s[-2]))
            elif kind == 'softmax':
                if not s or s[-1] < 2:
                    continue
                steps.append(('softmax', (i,), ())); shapes.append(s)
            elif kind == 'logsumexp':
                if not s or s[-1] < 2:
                    continue
                steps.append(('logsumexp', (i,), ())); shapes.append(s[:-1])
            elif kind == 'logdet_spd':
                # log det (v v^T + 2 I): symmetric positive definite, eigenvalues >= 2
                if len(s) < 2 or s[-2] > 6:
                    continue
                steps.append(('logdet_spd', (i,), ())); shapes.append(s[:-2])
            elif kind in ('inv_spd', 'solve_spd'):
                if len(s) < 2 or s[-2] > 5 or s[-2] < 2:
                    continue
                steps.append((kind, (i,), ())); shapes.append((*s[:-2], s[-2], s[-2]) if kind == 'inv_spd' else (*s[:-1], s[-1]))
            elif kind == 'attention':
                # value (n, H d) with H in {1, 2}: q = tanh(v), k = sin(v), v = v reshaped to (n, H, d)
                if len(s) != 2 or s[-1] % 2 != 0 or s[0] < 2:
                    continue
                H = int(rng.choice([1, 2]))
                steps.append(('attention', (i,), (H,))); shapes.append(s)
            elif kind == 'scatter':
                if len(s) != 1 or s[0] < 3:
                    continue
                n_upd = int(rng.integers(1, 4))
                cands = [j for j in range(1, len(shapes)) if len(shapes[j]) == 1 and shapes[j][0] >= n_upd]
                j = int(rng.choice(cands))
                idx = rng.integers(0, s[0], size=n_upd)
                steps.append(('scatter', (i, j), (idx, str(rng.choice(['set', 'add'])) if len(set(idx.tolist())) == n_upd else 'add')))
                shapes.append(s)
            elif kind in ('cumprod', 'cummax', 'prod', 'amin'):
                if not s or s[-1] < 2 or s[-1] > 8:
                    continue
                steps.append((kind, (i,), ())); shapes.append(s if kind in ('cumprod', 'cummax') else s[:-1])
            elif kind in ('minimum', 'maximum'):
                cands = [j for j in range(1, len(shapes)) if shapes[j] == s and j != i]
                if not cands:
                    continue
                steps.append((kind, (i, int(rng.choice(cands))), ())); shapes.append(s)
            elif kind == 'clip':
                steps.append(('clip', (i,), (-0.45, 0.7))); shapes.append(s)
            elif kind == 'layer_norm':
                if not s or s[-1] < 3:
                    continue
                steps.append(('layer_norm', (i,), ())); shapes.append(s)
            elif kind == 'where_data':
                cands = [j for j in range(1, len(shapes)) if shapes[j] == s]
                steps.append(('where_data', (i, int(rng.choice(cands))), ())); shapes.append(s)
            elif kind == 'abs_sqrt':
                steps.append(('abs_sqrt', (i,), ())); shapes.append(s)
            if int(np.prod(shapes[-1], dtype=int)) > 400 * max(n_in // N_IN, 1):     # keep the values small
                steps.pop(); shapes.pop()
                continue
            break
    return steps


def run(steps, xp, x):
    """Replays a program on a namespace (``folx_amd.numpy``, ``oracle.backend``, ``bruteforce.plain``)."""
    vals = [x]
    for op, src, static in steps:
        a = [vals[i] for i in src]
        if op == 'reshape':
            v = xp.reshape(a[0], static[0])
        elif op in _UNARY:
            v = getattr(xp, op)(a[0])
        elif op == 'divide' and len(a) == 2:
            v = xp.divide(a[0], xp.add(xp.square(a[1]), 1.5))     # a denominator that stays away from zero
        elif op in _BINARY or op in ('add', 'multiply'):
            v = getattr(xp, op)(a[0], a[1] if len(a) == 2 else static[0])
        elif op == 'transpose':
            v = xp.transpose(a[0], static[0])
        elif op == 'getitem':
            v = xp.getitem(a[0], static[0])
        elif op in ('sum', 'mean'):
            v = getattr(xp, op)(a[0], axis=static[0], keepdims=static[1])
        elif op == 'dot':
            v = xp.dot(a[0], static[0])
        elif op == 'concatenate':
            v = xp.concatenate([a[0], a[1]], axis=static[0])
        elif op == 'broadcast_to':
            v = xp.broadcast_to(a[0], static[0])
        elif op == 'flip':
            v = xp.flip(a[0], static[0])
        elif op == 'where':
            v = xp.where(static[0], a[0], a[1])
        elif op == 'cumsum':
            v = xp.cumsum(a[0], axis=static[0])
        elif op == 'amax':
            v = xp.amax(a[0], axis=static[0])
        elif op == 'take':
            v = xp.take(a[0], static[0], axis=static[1])
        elif op == 'lax_pad':
            v = xp.lax_pad(a[0], static[0], static[1])
        elif op == 'matmul_t':
            v = xp.matmul(a[0], xp.swapaxes(xp.tanh(a[1]), -1, -2))
        elif op == 'softmax':
            v = xp.softmax(xp.tanh(a[0]), axis=-1)
        elif op == 'logsumexp':
            v = xp.logsumexp(xp.tanh(a[0]), axis=-1)[0]
        elif op in ('inv_spd', 'solve_spd'):
            t = xp.tanh(a[0])
            m = t.shape[-2]
            A = xp.add(xp.matmul(t, xp.swapaxes(t, -1, -2)), 2.0 * np.eye(m, dtype=np.float32))
            v = xp.inv(A) if op == 'inv_spd' else xp.solve(A, xp.sin(a[0]))
        elif op == 'attention':
            n, w = a[0].shape
            H = static[0]
            q, k, vv = (xp.reshape(f(a[0]), (n, H, w // H)) for f in (xp.tanh, xp.sin, lambda z: z))
            v = xp.reshape(xp.multi_head_self_attention(q, k, vv), (n, w))
        elif op == 'scatter':
            v = xp.scatter(a[0], static[0], xp.getitem(xp.sin(a[1]), (slice(0, len(static[0])),)), static[1])
        elif op in ('cumprod', 'prod'):
            v = getattr(xp, op)(xp.add(xp.multiply(xp.tanh(a[0]), 0.5), 1.2), axis=-1)
        elif op in ('cummax', 'amin'):
            v = getattr(xp, op)(xp.sin(xp.multiply(a[0], 1.7)), axis=-1)
        elif op in ('minimum', 'maximum'):
            v = getattr(xp, op)(xp.sin(a[0]), xp.cos(a[1]))
        elif op == 'clip':
            v = xp.clip(xp.sin(a[0]), static[0], static[1])
        elif op == 'layer_norm':
            v = xp.layer_norm(xp.sin(a[0]), None, None, 1e-3)
        elif op == 'where_data':
            v = xp.where(xp.greater(xp.sin(xp.multiply(a[0], 2.3)), 0.05), xp.tanh(a[0]), xp.multiply(xp.cos(a[1]), 0.3))
        elif op == 'abs_sqrt':
            v = xp.sqrt(xp.add(xp.abs(xp.sin(xp.multiply(a[0], 1.3))), 0.3))
        elif op == 'logdet_spd':
            t = xp.tanh(a[0])
            m = t.shape[-2]
            v = xp.slogdet(xp.add(xp.matmul(t, xp.swapaxes(t, -1, -2)), 2.0 * np.eye(m, dtype=np.float32)))[1]
        else:
            raise KeyError(op)
        vals.append(v)
    return vals[-1]


USES_DETERMINANT = lambda steps: any(op == 'logdet_spd' for op, _, _ in steps)


def describe(steps):
    return ' ; '.join(f'{op}{src}' for op, src, _ in steps)

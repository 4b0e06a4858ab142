"""The per-rule cases of the reference's own layer tests (test/test_layers.py, the real-valued halves), each as a pair:
the function written with ``folx_amd.numpy`` and the same function in plain torch for the fp64 brute force
(test/laplacian_testcase.py:22-49).  One sample in, as in the reference; run on the CPU stand-ins and on the GPU by
``tests/test_reference_layers.py``."""

import numpy as np
import torch

from folx_amd import numpy as fnp

_rng = np.random.default_rng(2024)
X10 = _rng.normal(size=10).astype(np.float32)
X10B = _rng.normal(size=10).astype(np.float32)
X6 = _rng.normal(size=6).astype(np.float32)
_c = lambda v, t: torch.as_tensor(np.asarray(v), dtype=t.dtype)    # noqa: E731


def _elementwise():   # test/test_layers.py:38-61
    pairs = [('sin', fnp.sin, torch.sin), ('cos', fnp.cos, torch.cos), ('tanh', fnp.tanh, torch.tanh),
             ('exp', fnp.exp, torch.exp), ('square', fnp.square, torch.square), ('abs', fnp.abs, torch.abs),
             ('log_abs', lambda x: fnp.log(fnp.abs(x)), lambda x: torch.log(torch.abs(x))),
             ('sqrt_abs', lambda x: fnp.sqrt(fnp.abs(x)), lambda x: torch.sqrt(torch.abs(x)))]
    return {f'elementwise_{n}': (f, g, X10) for n, f, g in pairs}


def _binary():        # test/test_layers.py:63-117: both arguments, left only, right only
    ops = [('add', fnp.add, torch.add), ('subtract', fnp.subtract, torch.sub), ('multiply', fnp.multiply, torch.mul),
           ('divide', fnp.divide, torch.div)]
    out = {}
    x = np.stack([X10, X10B])
    for n, f, g in ops:
        out[f'binary_{n}_both'] = (lambda x, f=f: f(x[0], x[1]), lambda x, g=g: g(x[0], x[1]), x)
        out[f'binary_{n}_left'] = (lambda x, f=f: f(x, X10B), lambda x, g=g: g(x, _c(X10B, x)), X10)
        out[f'binary_{n}_right'] = (lambda x, f=f: f(X10B, x), lambda x, g=g: g(_c(X10B, x), x), X10)
    return out


def _elementwise_real():   # test/test_layers.py:695-716
    sp = torch.special
    pairs = [
        ('erf', fnp.erf, sp.erf), ('erfc', fnp.erfc, sp.erfc),
        ('erfinv_tanh', lambda z: fnp.erfinv(fnp.tanh(z)), lambda z: sp.erfinv(torch.tanh(z))),
        ('sinh', fnp.sinh, torch.sinh), ('cosh', fnp.cosh, torch.cosh), ('arcsinh', fnp.arcsinh, torch.asinh),
        ('arccosh', lambda z: fnp.arccosh(fnp.add(fnp.abs(z), 1.5)), lambda z: torch.acosh(torch.abs(z) + 1.5)),
        ('arctanh_tanh', lambda z: fnp.arctanh(fnp.tanh(z)), lambda z: torch.atanh(torch.tanh(z))),
        ('cbrt', fnp.cbrt, lambda z: torch.sign(z) * torch.abs(z) ** (1.0 / 3.0)),
        ('exp2', fnp.exp2, torch.exp2),
        ('gammaln', lambda z: fnp.gammaln(fnp.add(fnp.abs(z), 0.5)), lambda z: torch.lgamma(torch.abs(z) + 0.5)),
        ('digamma', lambda z: fnp.digamma(fnp.add(fnp.abs(z), 0.5)), lambda z: torch.digamma(torch.abs(z) + 0.5)),
        ('gelu_exact', lambda z: fnp.gelu(z, approximate=False), lambda z: torch.nn.functional.gelu(z)),
    ]
    return {f'real_{n}': (f, g, X6) for n, f, g in pairs}


def _piecewise():     # test/test_layers.py:718-733
    def t_rem(z):     # C-style remainder, as jax.lax.rem
        return z - 0.7 * torch.trunc(z / 0.7)

    pairs = [
        ('clip', lambda z: fnp.clip(z, -0.5, 0.5), lambda z: torch.clamp(z, -0.5, 0.5)),
        ('rem', lambda z: fnp.remainder(z, 0.7), t_rem),
        ('floor', lambda z: fnp.multiply(fnp.floor(fnp.multiply(z, 3.0)), z), lambda z: torch.floor(z * 3).detach() * z),
        ('ceil', lambda z: fnp.multiply(fnp.ceil(fnp.multiply(z, 3.0)), z), lambda z: torch.ceil(z * 3).detach() * z),
        ('round', lambda z: fnp.multiply(fnp.round(fnp.multiply(z, 3.0)), z), lambda z: torch.round(z * 3).detach() * z),
        ('cummax', lambda z: fnp.cummax(z, axis=0), lambda z: torch.cummax(z, 0).values),
        ('cummin', lambda z: fnp.cummin(z, axis=0), lambda z: torch.cummin(z, 0).values),
    ]
    return {f'piecewise_{n}': (f, g, X6) for n, f, g in pairs}


def _indexing():      # test/test_layers.py:747-761
    def t_dus(op, upd, start):
        out = op.clone()
        out[start:start + upd.shape[0]] = upd
        return out

    pairs = [
        ('stack_axis1', lambda z: fnp.stack([z, fnp.multiply(z, 2.0)], axis=1), lambda z: torch.stack([z, z * 2], dim=1)),
        ('stack_with_ones', lambda z: fnp.stack([z, np.ones(6, np.float32)], axis=0),
         lambda z: torch.stack([z, torch.ones(6, dtype=z.dtype)], dim=0)),
        ('unstack', lambda z: fnp.unstack(fnp.reshape(z, (2, 3)))[1], lambda z: z.reshape(2, 3)[1]),
        ('tile', lambda z: fnp.tile(fnp.reshape(z, (2, 3)), (2, 2)), lambda z: z.reshape(2, 3).repeat(2, 2)),
        ('copy', lambda z: fnp.multiply(fnp.copy(z), z), lambda z: z.clone() * z),
        ('update_slice_of_input', lambda z: fnp.dynamic_update_slice(z, fnp.square(fnp.getitem(z, slice(0, 2))), (3,)),
         lambda z: t_dus(z, z[:2] ** 2, 3)),
        ('update_slice_of_zeros', lambda z: fnp.dynamic_update_slice(np.zeros(8, np.float32), fnp.square(z), (3,)),
         lambda z: t_dus(torch.zeros(8, dtype=z.dtype), z ** 2, 2)),   # lax clamps the start: min(3, 8 - 6) = 2
    ]
    return {f'indexing_{n}': (f, g, X6) for n, f, g in pairs}


_W1 = _rng.normal(size=(4, 8)).astype(np.float32)
_W2 = _rng.normal(size=(4, 4, 8)).astype(np.float32)
X4 = _rng.normal(size=4).astype(np.float32)
X32 = _rng.normal(size=(2, 16)).astype(np.float32)

CASES = {
    'summation': (fnp.sum, torch.sum, X10),                                            # test/test_layers.py:25-36
    'cumprod_of_sin': (lambda z: fnp.cumprod(fnp.sin(z)), lambda z: torch.cumprod(torch.sin(z), 0), X6),   # :735-745
    'dot_of_two_inputs': (lambda x: fnp.vdot(x[0], x[1]), lambda x: torch.dot(x[0], x[1]), X32),           # :234-252
    'polynomial': (lambda x: fnp.add(fnp.dot(x, _W1), fnp.einsum('i,j,ijk->k', x, x, _W2)),                # :254-271
                   lambda x: x @ _c(_W1, x) + torch.einsum('i,j,ijk->k', x, x, _c(_W2, x)), X4),
    **_elementwise(), **_binary(), **_elementwise_real(), **_piecewise(), **_indexing(),
}

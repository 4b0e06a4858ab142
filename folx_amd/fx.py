"""A traced front door: ``forward_laplacian_torch(fn, sparsity_threshold)`` takes a model written with PLAIN TORCH
(one sample in, tensors out), traces it once per input shape into a graph of primitive operations and evaluates
that graph equation by equation through the rule registry -- what the reference does with a jaxpr
(``eval_jaxpr_with_forward_laplacian``, folx/interpreter.py:127-264: per equation, constants are evaluated
eagerly (:222-245), everything else looks its rule up under the primitive's name (:210-216), a primitive
without a rule gets the generic wrap with a warning, folx/wrapped_functions.py:597-618).

Here the trace is ``torch.fx`` (``make_fx`` on a CPU example: an ATen-level graph with concrete shapes, module
parameters lifted to graph constants) and an equation's rule is the ``folx_amd.numpy`` function of the same
meaning, which dispatches to the registry under the reference's primitive names; so a product meets the
LayerNorm in front of it and the activation behind it exactly as in a model written against
``folx_amd.numpy``.  The define-by-run front end stays the primary one; this is for models that exist as torch code."""

from __future__ import annotations

import logging
import operator

import numpy as np
import torch

from . import numpy as fnp
from .api import BatchedArray, FwdLaplArray
from .interpreter import ForwardLaplacianFn

aten = torch.ops.aten

# Named functions: the reference reaches its attention kernel through the NAME of a jitted function
# (``register_function('_multi_head_self_attention', ...)``, folx/experimental/pallas/attention/__init__.py:45, looked
# up by ``eval_pjit``, folx/interpreter.py:186-200).  The torch counterpart is a library operation: while a model is
# being traced the function below records ONE node, which the graph evaluation hands to the rule registered under the
# same key; outside a trace it is the plain differentiable arithmetic.
_LIB = torch.library.Library('folx_amd', 'DEF')
_LIB.define('multi_head_self_attention(Tensor q, Tensor k, Tensor v) -> Tensor')
_TRACING = [False]


def _mhsa_math(q, k, v):
    p = torch.softmax(torch.einsum('ihd,jhd->hij', q, k), dim=-1)
    return torch.einsum('hij,jhd->ihd', p, v)


_LIB.impl('multi_head_self_attention', _mhsa_math, 'CompositeExplicitAutograd')


def multi_head_self_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """``softmax(q k^T) v`` for per-sample tensors ``(n, heads, d)`` (no ``1 / sqrt(d)`` inside, as in the reference's
    ``folx.experimental.pallas.attention.multi_head_self_attention``): in a model traced by
    ``forward_laplacian_torch`` this is one equation and runs on the attention rule's kernel."""
    if _TRACING[0]:
        return torch.ops.folx_amd.multi_head_self_attention(q, k, v)
    return _mhsa_math(q, k, v)



def _is_t(v):
    from .wrapped_functions import Deferred

    return isinstance(v, (FwdLaplArray, BatchedArray, Deferred))


def _const(v):
    """Graph constants travel as numpy (float32 for floating point), python scalars as they are."""
    if isinstance(v, torch.Tensor):
        a = v.detach().cpu().numpy()
        return a.astype(np.float32) if np.issubdtype(a.dtype, np.floating) else a
    return v


def _shape(v):
    return tuple(fnp._shape(v)) if _is_t(v) else tuple(np.shape(v))


def _dims(d, nd):
    if d is None or (isinstance(d, (list, tuple)) and len(d) == 0):
        return tuple(range(nd))
    return tuple(int(i) % nd for i in (d if isinstance(d, (list, tuple)) else (d,)))


def _reduce(fn):
    def rule(a, dim=None, keepdim=False, dtype=None):
        nd = len(_shape(a))
        if nd == 0:
            return a
        return fn(a, axis=_dims(dim, nd), keepdims=bool(keepdim))

    return rule


def _view(a, shape):
    shape = [int(n) for n in shape]
    if -1 in shape:
        known = int(np.prod([n for n in shape if n != -1], dtype=int))
        shape[shape.index(-1)] = int(np.prod(_shape(a), dtype=int)) // max(known, 1)
    return fnp.reshape(a, tuple(shape))


def _expand(a, sizes, implicit=False):
    s = _shape(a)
    sizes = [int(n) for n in sizes]
    lead = len(sizes) - len(s)
    target = tuple(s[i - lead] if n == -1 else n for i, n in enumerate(sizes))
    if target == s:
        return a
    if len(target) == len(s):   # size-1 axes grow: a product with ones keeps it one rule (and sparse rows sparse)
        return fnp.multiply(a, np.ones(target, dtype=np.float32))
    return fnp.broadcast_to(a, target) if all(x == y for x, y in zip(target[lead:], s)) else \
        fnp.multiply(fnp.reshape(a, (1,) * lead + s), np.ones(target, dtype=np.float32))


def _slice(a, dim=0, start=None, end=None, step=1):
    nd = len(_shape(a))
    dim = dim % nd
    n = _shape(a)[dim]
    end = None if end is None or end >= n else end     # ATen passes sys.maxsize for "to the end"
    return fnp.getitem(a, (*([slice(None)] * dim), slice(start, end, step)))


def _select(a, dim, index):
    nd = len(_shape(a))
    return fnp.getitem(a, (*([slice(None)] * (dim % nd)), int(index)))


def _index(a, indices):
    idx = tuple(slice(None) if i is None else np.asarray(i) for i in indices)
    return fnp.getitem(a, idx)


def _pow_scalar(a, e):
    if float(e) == int(e):
        return fnp.integer_pow(a, int(e))
    return fnp.power(a, float(e))


def _scaled(v, alpha):
    return v if alpha == 1 else fnp.multiply(v, float(alpha))


def _addmm(bias, a, b, beta=1, alpha=1):
    return fnp.add(_scaled(fnp.matmul(a, b), alpha), _scaled(bias, beta))


def _layer_norm(a, normalized_shape, weight, bias, eps):
    assert len(normalized_shape) == 1, 'native_layer_norm: only the last axis is normalised by the LayerNorm rule'
    return fnp.layer_norm(a, weight, bias, float(eps)), None, None


def _softplus(a, beta=1.0, threshold=20.0):
    if float(beta) == 1.0:
        return fnp.softplus(a)
    return fnp.multiply(fnp.softplus(fnp.multiply(a, float(beta))), 1.0 / float(beta))


def _squeeze(a, dims=None):
    s = _shape(a)
    ds = _dims(dims, len(s)) if dims is not None else tuple(range(len(s)))
    return fnp.reshape(a, tuple(n for i, n in enumerate(s) if not (i in ds and n == 1)))


def _max_dim(arg_fn, val_fn):
    def rule(a, dim, keepdim=False):
        v, i = val_fn(a, axis=int(dim)), arg_fn(a, axis=int(dim))
        if keepdim:
            v, i = fnp.expand_dims(v, int(dim)), np.expand_dims(np.asarray(i), int(dim)) if not _is_t(i) else i
        return v, i

    return rule


class _OnDemand:
    """An output of a multi-output operation that is only computed when the graph reads it."""

    def __init__(self, make):
        self.make = make


def _scan_with_indices(scan_fn, arg_fn):
    """``cummax`` / ``cummin``: values from the scan; indices (no derivatives) = the arg-extremum over each prefix,
    from an (n, n) masked copy, built only if the graph reads them."""
    def rule(a, dim):
        s = _shape(a)
        ax = int(dim) % len(s)
        n = s[ax]

        def indices():
            v = fnp.stop_gradient(a)
            big = np.float32(np.finfo(np.float32).max) * (1.0 if arg_fn is fnp.argmin else -1.0)
            keep = np.tril(np.ones((n, n), dtype=bool)).reshape((n,) + (1,) * (len(s) - 1 - ax) + (n,))
            rows = fnp.expand_dims(fnp.moveaxis(v, ax, -1), ax)            # (..., 1, ..., n): prefix i reads entries <= i
            full = fnp.where(keep, rows, big)
            return arg_fn(full, axis=-1)

        return scan_fn(a, axis=ax), _OnDemand(indices)

    return rule


def _item(a, i):
    v = a[i]
    return v.make() if isinstance(v, _OnDemand) else v


def _clamp(a, lo=None, hi=None):
    return fnp.clip(a, lo, hi)


def _identity(a, *_, **__):
    return a


# ATen operation -> the function of the same meaning (which finds its rule in the registry)
RULES = {
    aten.add.Tensor: lambda a, b, alpha=1: fnp.add(a, _scaled(b, alpha)),
    aten.add.Scalar: lambda a, b, alpha=1: fnp.add(a, float(b) * float(alpha)),
    aten.sub.Tensor: lambda a, b, alpha=1: fnp.subtract(a, _scaled(b, alpha)),
    aten.sub.Scalar: lambda a, b, alpha=1: fnp.subtract(a, float(b) * float(alpha)),
    aten.rsub.Scalar: lambda a, b, alpha=1: fnp.subtract(float(b), _scaled(a, alpha)),
    aten.mul.Tensor: fnp.multiply, aten.mul.Scalar: lambda a, b: fnp.multiply(a, float(b)),
    aten.div.Tensor: fnp.divide, aten.div.Scalar: lambda a, b: fnp.multiply(a, 1.0 / float(b)),
    aten.neg.default: fnp.negative, aten.reciprocal.default: fnp.reciprocal,
    aten.tanh.default: fnp.tanh, aten.sin.default: fnp.sin, aten.cos.default: fnp.cos, aten.exp.default: fnp.exp,
    aten.log.default: fnp.log, aten.sqrt.default: fnp.sqrt, aten.rsqrt.default: fnp.rsqrt,
    aten.sigmoid.default: fnp.sigmoid, aten.silu.default: fnp.silu, aten.relu.default: fnp.relu,
    aten.gelu.default: lambda a, approximate='none': fnp.gelu(a, approximate=(approximate == 'tanh')),
    aten.erf.default: fnp.erf, aten.erfc.default: fnp.erfc, aten.erfinv.default: fnp.erf_inv, aten.abs.default: fnp.abs,
    aten.expm1.default: fnp.expm1, aten.log1p.default: fnp.log1p, aten.sinh.default: fnp.sinh,
    aten.cosh.default: fnp.cosh, aten.tan.default: fnp.tan, aten.atan.default: fnp.arctan,
    aten.asin.default: fnp.arcsin, aten.acos.default: fnp.arccos, aten.asinh.default: fnp.arcsinh,
    aten.acosh.default: fnp.arccosh, aten.atanh.default: fnp.arctanh, aten.exp2.default: fnp.exp2,
    aten.lgamma.default: fnp.lgamma, aten.digamma.default: fnp.digamma, aten.atan2.default: fnp.arctan2,
    aten.softplus.default: _softplus, aten.elu.default: lambda a, alpha=1.0, scale=1.0, input_scale=1.0: fnp.elu(a, alpha),
    aten.leaky_relu.default: lambda a, negative_slope=0.01: fnp.leaky_relu(a, negative_slope),
    aten.pow.Tensor_Scalar: _pow_scalar, aten.pow.Tensor_Tensor: fnp.power, aten.pow.Scalar: lambda b, e: fnp.power(float(b), e),
    aten.square.default: fnp.square,
    aten.mm.default: fnp.matmul, aten.bmm.default: fnp.matmul, aten.matmul.default: fnp.matmul, aten.addmm.default: _addmm,
    aten.dot.default: fnp.vdot, aten.mv.default: fnp.matmul,
    aten.t.default: lambda a: a if len(_shape(a)) < 2 else fnp.swapaxes(a, -1, -2),
    aten.transpose.int: lambda a, d0, d1: fnp.swapaxes(a, int(d0), int(d1)),
    aten.permute.default: lambda a, dims: fnp.transpose(a, [int(d) for d in dims]),
    aten.view.default: _view, aten.reshape.default: _view, aten._unsafe_view.default: _view,
    aten.expand.default: _expand,
    aten.unsqueeze.default: lambda a, dim: fnp.expand_dims(a, int(dim)),
    aten.squeeze.dim: lambda a, dim: _squeeze(a, (dim,)), aten.squeeze.dims: _squeeze, aten.squeeze.default: _squeeze,
    aten.slice.Tensor: _slice, aten.select.int: _select, aten.index.Tensor: _index,
    aten.cat.default: lambda ts, dim=0: fnp.concatenate(list(ts), axis=int(dim)),
    aten.stack.default: lambda ts, dim=0: fnp.stack(list(ts), axis=int(dim)),
    aten.flip.default: lambda a, dims: fnp.flip(a, tuple(int(d) for d in dims)) if len(dims) > 1 else fnp.flip(a, int(dims[0])),
    aten.sum.default: _reduce(fnp.sum), aten.sum.dim_IntList: _reduce(fnp.sum),
    aten.mean.default: _reduce(fnp.mean), aten.mean.dim: _reduce(fnp.mean),
    aten.amax.default: lambda a, dim=(), keepdim=False: _fold_axes(fnp.amax, a, dim, keepdim),
    aten.amin.default: lambda a, dim=(), keepdim=False: _fold_axes(fnp.amin, a, dim, keepdim),
    aten.max.dim: _max_dim(fnp.argmax, fnp.amax), aten.min.dim: _max_dim(fnp.argmin, fnp.amin),
    aten.prod.dim_int: lambda a, dim, keepdim=False, dtype=None: _fold_axes(fnp.prod, a, (dim,), keepdim),
    aten.cumsum.default: lambda a, dim, dtype=None: fnp.cumsum(a, axis=int(dim)),
    aten.cumprod.default: lambda a, dim, dtype=None: fnp.cumprod(a, axis=int(dim)),
    aten.cummax.default: _scan_with_indices(fnp.cummax, fnp.argmax), aten.cummin.default: _scan_with_indices(fnp.cummin, fnp.argmin),
    aten.unbind.int: lambda a, dim=0: tuple(_select(a, dim, i) for i in range(_shape(a)[int(dim) % len(_shape(a))])),
    aten._softmax.default: lambda a, dim, half=False: fnp.softmax(a, axis=int(dim)),
    aten._log_softmax.default: lambda a, dim, half=False: fnp.log_softmax(a, axis=int(dim)),
    aten.logsumexp.default: lambda a, dim, keepdim=False: _logsumexp(a, dim, keepdim),
    aten.native_layer_norm.default: _layer_norm,
    aten.where.self: fnp.where,
    aten.gt.Scalar: fnp.greater, aten.gt.Tensor: fnp.greater, aten.ge.Scalar: fnp.greater_equal, aten.ge.Tensor: fnp.greater_equal,
    aten.lt.Scalar: fnp.less, aten.lt.Tensor: fnp.less, aten.le.Scalar: fnp.less_equal, aten.le.Tensor: fnp.less_equal,
    aten.eq.Scalar: fnp.equal, aten.eq.Tensor: fnp.equal, aten.ne.Scalar: fnp.not_equal, aten.ne.Tensor: fnp.not_equal,
    aten.logical_and.default: fnp.logical_and, aten.logical_or.default: fnp.logical_or, aten.logical_not.default: fnp.logical_not,
    aten.clamp.default: _clamp, aten.clamp_min.default: lambda a, lo: fnp.clip(a, lo, None),
    aten.clamp_max.default: lambda a, hi: fnp.clip(a, None, hi),
    aten.minimum.default: fnp.minimum, aten.maximum.default: fnp.maximum,
    aten.clone.default: _identity, aten.alias.default: _identity, aten.contiguous.default: _identity,
    aten._to_copy.default: _identity, aten.lift_fresh_copy.default: _identity,
    aten.detach.default: fnp.stop_gradient,
    aten._linalg_slogdet.default: lambda A: (*fnp.slogdet(A), None, None),
    aten._linalg_det.default: lambda A: (fnp.det(A), None, None),
    aten.linalg_inv_ex.default: lambda A, check_errors=False: (fnp.inv(A), None),
    aten._linalg_solve_ex.default: lambda A, B, left=True, check_errors=False: (fnp.solve(A, B), None, None, None),
    operator.getitem: _item,
    aten.sign.default: fnp.sign, aten.sgn.default: fnp.sign,
    # a constant that only borrows the SHAPE of a data tensor (the seed of a gradient taken inside the function, ...)
    aten.ones_like.default: lambda a, **_: np.ones(_shape(a), np.float32),
    aten.zeros_like.default: lambda a, **_: np.zeros(_shape(a), np.float32),
    aten.full_like.default: lambda a, value, **_: np.full(_shape(a), float(value), np.float32),
    aten.new_ones.default: lambda a, size, **_: np.ones(tuple(int(n) for n in size), np.float32),
    aten.new_zeros.default: lambda a, size, **_: np.zeros(tuple(int(n) for n in size), np.float32),
    aten.new_full.default: lambda a, size, value, **_: np.full(tuple(int(n) for n in size), float(value), np.float32),
    aten.index_select.default: lambda a, dim, index: fnp.take(a, np.asarray(index), axis=int(dim)),
    aten.take.default: lambda a, index: fnp.take(a, np.asarray(index)),
    aten.squeeze_.dim: lambda a, dim: _squeeze(a, (dim,)), aten.unsqueeze_.default: lambda a, dim: fnp.expand_dims(a, int(dim)),
    aten._safe_softmax.default: lambda a, dim, dtype=None: fnp.softmax(a, axis=int(dim)),
    torch.ops.folx_amd.multi_head_self_attention.default: fnp.multi_head_self_attention,
}


def _amax_values(a, dims=(), keepdim=False):
    s = _shape(a)
    axes = _dims(dims, len(s))
    return fnp.amax_const(a, axes, keepdims=bool(keepdim))


def _fold_axes(fn, a, dims, keepdim):
    s = _shape(a)
    axes = sorted(_dims(dims, len(s)), reverse=True)
    out = a
    for ax in axes:
        out = fn(out, axis=ax)
    if keepdim:
        out = fnp.reshape(out, tuple(1 if i in axes else n for i, n in enumerate(s)))
    return out


def _logsumexp(a, dims, keepdim):
    s = _shape(a)
    axes = _dims(dims, len(s))
    assert len(axes) == 1, 'logsumexp: one axis'
    out = fnp.logsumexp(a, axis=axes[0])[0]
    return fnp.expand_dims(out, axes[0]) if keepdim else out


def _generic(target):
    """An ATen operation without an entry above: the generic rule built from the operation itself, with the warning
    the reference gives for a primitive outside its registry (folx/wrapped_functions.py:609-614)."""
    def rule(*args, **kwargs):
        logging.warning(f'{target} has no forward-Laplacian rule; the following call computes the full Hessian of the operation')
        return fnp.call(lambda *a: target(*a, **kwargs), *args)

    return rule


def _tree(v, fn):
    if isinstance(v, (list, tuple)):
        return type(v)(_tree(t, fn) for t in v)
    if isinstance(v, dict):
        return {k: _tree(t, fn) for k, t in v.items()}
    return fn(v)


def _any_triplet(v):
    if isinstance(v, (list, tuple)):
        return any(_any_triplet(t) for t in v)
    if isinstance(v, dict):
        return any(_any_triplet(t) for t in v.values())
    return _is_t(v)


def fold_constants(gm: torch.fx.GraphModule):
    """Every equation whose inputs are all constants, evaluated once by torch itself on the host (the reference binds
    such equations eagerly while it interprets, folx/interpreter.py:222-245): node -> numpy array / scalar / tuple."""
    env = {}
    look = lambda a: env[a] if isinstance(a, torch.fx.Node) else a
    is_const = lambda a: not isinstance(a, torch.fx.Node) or a in env

    def all_const(v):
        if isinstance(v, (list, tuple)):
            return all(all_const(t) for t in v)
        if isinstance(v, dict):
            return all(all_const(t) for t in v.values())
        return is_const(v)

    for node in gm.graph.nodes:
        if node.op == 'get_attr':
            obj = gm
            for part in node.target.split('.'):
                obj = getattr(obj, part)
            env[node] = obj.detach() if isinstance(obj, torch.Tensor) else obj
        elif node.op == 'call_function' and all_const(node.args) and all_const(node.kwargs):
            args = torch.fx.node.map_arg(node.args, look)
            kwargs = torch.fx.node.map_arg(node.kwargs, look)
            with torch.no_grad():
                env[node] = node.target(*args, **kwargs)
    return {n: _tree(v, _const) for n, v in env.items()}


_DEVICE_CONST_MIN = 256   # constants of at least this many floats live on the device between evaluations


def evaluate_graph(gm: torch.fx.GraphModule, inputs, consts=None):
    """One pass over the equations of a traced graph (folx/interpreter.py:218-264): constant equations come from
    ``fold_constants``, the others go through ``RULES``."""
    env = dict(fold_constants(gm) if consts is None else consts)
    it = iter(inputs)
    look = lambda a: env[a] if isinstance(a, torch.fx.Node) else a
    for node in gm.graph.nodes:
        if node in env:
            continue
        if node.op == 'placeholder':
            env[node] = next(it)
        elif node.op == 'call_function':
            args = torch.fx.node.map_arg(node.args, look)
            kwargs = torch.fx.node.map_arg(node.kwargs, look)
            kwargs = {k: v for k, v in kwargs.items() if k not in ('dtype', 'device', 'layout', 'pin_memory', 'memory_format')}
            rule = RULES.get(node.target) or _generic(node.target)
            if node.target is aten.amax.default and node.users and all(u.target is aten.detach.default for u in node.users):
                rule = _amax_values   # max(...).detach(): the shift of a softmax / logsumexp carries no derivatives
            try:
                env[node] = rule(*args, **kwargs)
            except Exception:
                logging.error(f'forward Laplacian of {node.format_node()} failed')   # folx/interpreter.py:254-257
                raise
        elif node.op == 'output':
            return torch.fx.node.map_arg(node.args[0], look)
        else:
            raise NotImplementedError(f'graph node {node.op}')
    raise RuntimeError('graph without an output')


class TracedForwardLaplacian(ForwardLaplacianFn):
    """``forward_laplacian_torch(fn, thr)``: ``f(x)`` takes one sample, ``f.batched(x)`` walkers, as for
    ``forward_laplacian``; the torch function is traced once per combination of input shapes, its constant
    equations are evaluated then, and the larger constants (weights) are uploaded once per device."""

    def __init__(self, fn, sparsity_threshold):
        self.torch_fn = fn
        self.graphs = {}
        self.constants = {}
        super().__init__(self._run, sparsity_threshold)

    def _graph(self, shapes):
        gm = self.graphs.get(shapes)
        if gm is None:
            from torch.fx.experimental.proxy_tensor import make_fx

            with torch.no_grad():
                examples = [torch.zeros(s, dtype=torch.float32) + 0.5 for s in shapes]
                _TRACING[0] = True
                try:
                    gm = self.graphs[shapes] = make_fx(self.torch_fn)(*examples)
                finally:
                    _TRACING[0] = False
            self.constants[shapes] = fold_constants(gm)
        return gm

    def _constants(self, shapes, device):
        key = (shapes, str(device))
        hit = self.constants.get(key)
        if hit is None:
            def place(v):
                if (isinstance(v, np.ndarray) and v.dtype == np.float32 and v.size >= _DEVICE_CONST_MIN
                        and device.type != 'cpu'):
                    return torch.as_tensor(np.ascontiguousarray(v)).to(device)
                return v
            hit = self.constants[key] = {n: _tree(v, place) for n, v in self.constants[shapes].items()}
        return hit

    def _run(self, *lapl_args):
        shapes = tuple(tuple(a.shape) for a in lapl_args)
        gm = self._graph(shapes)
        return evaluate_graph(gm, lapl_args, self._constants(shapes, lapl_args[0].x.device))

    def invalidate(self):
        """Forget the traces (and the constants folded from them): the next call traces again, e.g. after the
        parameters of a traced module have changed."""
        self.graphs.clear()
        self.constants.clear()


def forward_laplacian_torch(fn, sparsity_threshold: int | float = 0) -> TracedForwardLaplacian:
    """The traced counterpart of ``forward_laplacian`` for a function (or ``torch.nn.Module``) written with torch:
    ``fn(*tensors)`` maps ONE sample to a tensor or a tuple / list / dict of tensors; every tensor argument is
    differentiated (one index space, in argument order)."""
    return TracedForwardLaplacian(fn, sparsity_threshold)

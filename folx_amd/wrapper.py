"""Rules built from a function instead of written by hand (folx/wrapper.py:73-176).

``wrap_forward_laplacian(fn)`` turns a function of per-walker arrays into a forward-Laplacian
rule::

    y = fn(x),   J_y[p] = J_f(x) J_x[p],   lap_y = J_f(x) lap_x + sum_p J_x[p]^T H_f(x) J_x[p]

(folx/wrapper.py:118-125).  The reference takes ``J_f`` and ``H_f`` from jax's autodiff; here
``fn`` is written with torch and its derivatives come from ``torch.func`` in forward mode:
``jvp`` for ``J_f t`` and ``jvp`` of ``jvp`` for ``t^T H_f t`` (no Hessian is ever formed), mapped
over the Jacobian rows and the walkers with ``torch.func.vmap``.

This is the ONE rule whose arithmetic does not run in ``libfolx_hip.so``: what it computes is
defined by the caller's function alone, so it runs wherever PyTorch runs that function (on the
GPU, through PyTorch's kernels).  Nothing that ``folx_amd`` registers by itself goes through it;
it serves functions and primitives that have no hand-written rule (``register_function(name,
wrap_forward_laplacian(fn))``, ``get_laplacian(fn, wrap_if_missing=True)``).  The Jacobians
are taken dense, as the reference's full-Hessian path does past the sparsity threshold.
"""

from __future__ import annotations

from typing import Any, Callable

import numpy as np
import torch

from .api import BatchedArray, FunctionFlags, FwdJacobian, FwdLaplArray

__all__ = ['wrap_forward_laplacian', 'warp_without_fwd_laplacian', 'wrap_elementwise', 'custom_jvp']


def _is(a):
    return isinstance(a, FwdLaplArray)


def _force(a):
    from .wrapped_functions import Deferred, force

    return force(a) if isinstance(a, Deferred) else a


def _device_of(args):
    for a in args:
        if _is(a):
            return a.x.device
        if isinstance(a, BatchedArray):
            return a.data.device
    return None


def _dense_rows(t: FwdLaplArray, P: int) -> torch.Tensor:
    """Dense Jacobian (P, B, *shape): a sparse one is materialised, missing trailing rows are zero."""
    J = t.jacobian.dense_array
    if J.shape[0] < P:
        pad = J.new_zeros((P - J.shape[0], *J.shape[1:]))
        J = torch.cat([J, pad], dim=0)
    return J


class _HookJacobian:
    """What a ``custom_jac_hessian_jac`` hook sees of one argument's Jacobian: dense rows ``data (P, ...)``."""

    __slots__ = ('data', 'x0_idx')

    def __init__(self, data):
        self.data, self.x0_idx = data, None

    @property
    def weak(self):
        return False

    @property
    def dense_array(self):
        return self.data


class _HookArgs:
    """Per-position view of the derivative-carrying arguments handed to a ``custom_jac_hessian_jac`` hook
    (the fields of folx/api.py:348-409 that such hooks read)."""

    def __init__(self, xs, Js, laps):
        self.x = tuple(xs)
        self.jacobian = tuple(_HookJacobian(j) for j in Js)
        self.laplacian = tuple(laps)

    def __len__(self):
        return len(self.x)


def _tree_map(f, tree, *rest):
    if isinstance(tree, (tuple, list)):
        return type(tree)(_tree_map(f, t, *[r[i] for r in rest]) for i, t in enumerate(tree))
    return f(tree, *rest)


class custom_jvp:
    """A torch function with a derivative rule of the caller's own, spelled like ``jax.custom_jvp``::

        @folx_amd.custom_jvp
        def f(x): ...
        @f.defjvp
        def f_jvp(primals, tangents): return f(*primals), <J_f tangents>

    Called with forward-Laplacian triplets it is evaluated by the generic rule with ``f_jvp`` in place of the
    automatic ``J_f t`` -- the Jacobian and ``J_f lap`` come from the rule, ``t^T H_f t`` from its forward-mode
    derivative -- as the reference evaluates a ``custom_jvp_call`` equation (folx/interpreter.py:202-208,
    test/test_customjvp.py).  ``tangents`` holds zeros for the arguments that carry no derivatives.  Called with
    anything else it is the plain function; under the trace of ``forward_laplacian_torch`` it raises, because the
    trace would keep the function's operations and drop the rule."""

    def __init__(self, fn):
        self.fn = fn
        self.jvp_rule = None
        self.__name__ = getattr(fn, '__name__', 'custom_jvp')
        self._rule = None

    def defjvp(self, rule):
        self.jvp_rule = rule
        return rule

    def __call__(self, *args, **kwargs):
        from .numpy import current_threshold
        from .wrapped_functions import Deferred

        if not any(isinstance(a, (FwdLaplArray, Deferred)) for a in args):
            from .fx import _TRACING

            if _TRACING[0]:   # the trace would record the function's own operations and lose the rule
                raise NotImplementedError(f'{self.__name__}: a custom_jvp function cannot be traced by '
                                          'forward_laplacian_torch; call it under forward_laplacian')
            return self.fn(*args, **kwargs)
        if self.jvp_rule is None:
            raise AttributeError(f'no derivative rule was given for {self.__name__} (defjvp)')
        if self._rule is None:
            self._rule = wrap_forward_laplacian(self)
        return self._rule(args, kwargs, current_threshold())


def wrap_forward_laplacian(
    fn: Callable,
    in_axes=None,
    flags: FunctionFlags = FunctionFlags.GENERAL,
    name: str | None = None,
    index_static_args=None,
    custom_jac_hessian_jac=None,
):
    """folx/wrapper.py:73-138.  ``fn(*arrays, **kwargs)`` sees ONE walker: torch tensors without
    the walker axis where the rule is given ``FwdLaplArray`` / ``BatchedArray`` arguments, and the
    other arguments (numpy arrays, scalars, anything else) as they are.  It returns a tensor or a
    tuple / list of tensors.

    ``flags``: ``LINEAR`` skips the second-order term, as in the reference; the other flags
    choose cheaper forms of the same term there and change nothing here.  ``in_axes`` and
    ``index_static_args`` (which axes / arguments the reference may leave out of the Hessian) do
    not change the result and are accepted for compatibility -- except that ``in_axes`` decides what
    the hook below sees.

    ``custom_jac_hessian_jac(args, extra_args, merge, materialize_idx)`` is the reference's hook for
    a hand-written second-order term ``tr(J^T H_f J)`` (folx/api.py:434-441, called at
    folx/hessian.py:516-517): when given, the automatic ``t^T H_f t`` is not formed and the hook's
    result is added to ``J_f lap`` instead.  It is called as in the reference, once per position
    that ``in_axes`` maps over: ``in_axes=None`` shows it whole per-walker arrays, ``in_axes=()`` one
    element at a time, an int or tuple of axes the slices along those axes.  ``args`` has ``.x``,
    ``.jacobian`` (objects with ``.data`` of shape ``(P, ...)`` and ``.x0_idx = None``: the Jacobians
    are dense here) and ``.laplacian``, one entry per argument that carries derivatives;
    ``extra_args`` are the other arguments, ``merge(xs, extra_args)`` puts both back in call
    order; ``materialize_idx`` is always ``None`` (dense rows).  The result is a tensor, or a tree
    of tensors, with as many entries as the function's output has at those positions."""
    linear = (flags & FunctionFlags.LINEAR) == FunctionFlags.LINEAR or custom_jac_hessian_jac is not None
    if isinstance(in_axes, int):
        in_axes = (in_axes,)
    label = name or getattr(fn, '__name__', 'wrapped')

    def new_fn(args: tuple, kwargs: dict[str, Any], sparsity_threshold: int):
        from torch.func import jvp, vmap

        args = tuple(_force(a) for a in args)
        dev = _device_of(args)
        lapl_pos = [i for i, a in enumerate(args) if _is(a)]
        bat_pos = [i for i, a in enumerate(args) if isinstance(a, BatchedArray)]

        def const(a):
            if isinstance(a, np.ndarray) and dev is not None and a.dtype.kind == 'f':
                return torch.as_tensor(np.ascontiguousarray(a, dtype=np.float32), device=dev)
            return a

        consts = [None if (i in lapl_pos or i in bat_pos) else const(a) for i, a in enumerate(args)]

        def merged(xs, bs):
            full = list(consts)
            for i, x in zip(lapl_pos, xs):
                full[i] = x
            for i, b in zip(bat_pos, bs):
                full[i] = b
            return full

        plain = fn.fn if isinstance(fn, custom_jvp) else fn

        def call(xs, bs):
            return plain(*merged(xs, bs), **kwargs)

        def pushforward(g, xw, tv, bw):
            """``J_f t``: forward mode through ``g``, or the caller's rule for a ``custom_jvp`` function."""
            if not isinstance(fn, custom_jvp):
                return jvp(g, xw, tv)[1]
            primals = merged(xw, bw)
            tangents = [torch.zeros_like(v) if isinstance(v, torch.Tensor) else 0.0 for v in primals]
            for i, t in zip(lapl_pos, tv):
                tangents[i] = t
            return fn.jvp_rule(tuple(primals), tuple(tangents), **kwargs)[1]

        bvals = tuple(args[i].data for i in bat_pos)
        if not lapl_pos:  # nothing carries derivatives: a plain forward pass (folx/wrapper.py:112-114)
            if not bat_pos:
                return call((), ())
            out = vmap(lambda bs: call((), bs))(bvals)
            return _tree_map(lambda t: BatchedArray(t.to(torch.float32)) if t.is_floating_point() else BatchedArray(t),
                             out)

        ts = [args[i] for i in lapl_pos]
        P = max(t.jacobian.max_n + (1 if t.jacobian.weak else 0) for t in ts)
        xs = tuple(t.x for t in ts)                                   # (B, *shape)
        Js = tuple(_dense_rows(t, P).transpose(0, 1) for t in ts)     # (B, P, *shape)
        laps = tuple(t.laplacian for t in ts)

        extra_pos = [i for i in range(len(args)) if i not in lapl_pos]

        def hook_term(xw, Jw, lw, bw, y):
            """the caller's tr(J^T H_f J), evaluated position by position as ``in_axes`` says"""
            extra = tuple(bw[bat_pos.index(i)] if i in bat_pos else consts[i] for i in extra_pos)

            def merge(xs, ex):
                full = [None] * len(args)
                for i, v in zip(lapl_pos, xs):
                    full[i] = v
                for i, v in zip(extra_pos, ex):
                    full[i] = v
                return tuple(full)

            def at_position(xs, Js, ls):
                res = custom_jac_hessian_jac(_HookArgs(xs, Js, ls), extra, merge, None)
                leaves = []
                _tree_map(lambda t: leaves.append(torch.as_tensor(t).reshape(-1)), res)
                return torch.cat(leaves) if len(leaves) != 1 else leaves[0]

            Js = tuple(Jw)   # (P, *shape) per walker
            if in_axes is None:
                flat = at_position(xw, Js, lw)
            else:
                # positions = the axes NOT named by in_axes, the same for every argument; the hook is mapped over them
                nd = xw[0].dim()
                keep = sorted(a % nd for a in in_axes) if nd else []
                other = [a for a in range(nd) if a not in keep]
                mv = lambda t, lead: t.permute(*range(lead), *[lead + a for a in other], *[lead + a for a in keep]).reshape(
                    *t.shape[:lead], -1, *[t.shape[lead + a] for a in keep])
                xs_ = tuple(mv(t, 0) for t in xw)
                Js_ = tuple(mv(t, 1) for t in Js)
                ls_ = tuple(mv(t, 0) for t in lw)
                flat = vmap(at_position, in_dims=(0, 1, 0))(xs_, Js_, ls_).reshape(-1)
            leaves = []
            _tree_map(lambda t: leaves.append(t), y)
            total = sum(t.numel() for t in leaves)
            if flat.numel() == 1 and total != 1:       # one number for every output entry (e.g. a term that is zero)
                flat = flat.expand(total)
            assert flat.numel() == total, (f'custom_jac_hessian_jac returned {flat.numel()} values for an output of '
                                           f'{total} entries')
            outs, off = [], 0
            for t in leaves:
                outs.append(flat[off:off + t.numel()].reshape(t.shape))
                off += t.numel()
            it = iter(outs)
            return _tree_map(lambda t: next(it), y)

        def per_walker(xw, Jw, lw, bw):
            g = lambda *z: call(z, bw)  # noqa: E731
            first = lambda tv: pushforward(g, xw, tv, bw)  # noqa: E731   J_f t
            y = g(*xw)
            Jy = vmap(first)(Jw)
            lap = first(lw)
            if custom_jac_hessian_jac is not None:
                lap = _tree_map(lambda l, q: l + q, lap, hook_term(xw, Jw, lw, bw, y))
            elif not linear:
                second = lambda tv: jvp(lambda *z: pushforward(g, z, tv, bw), xw, tv)[1]  # noqa: E731   t^T H_f t
                quad = vmap(second)(Jw)
                lap = _tree_map(lambda l, q: l + q.sum(0), lap, quad)
            return y, Jy, lap

        y, Jy, lap = vmap(per_walker)(xs, Js, laps, bvals)

        def pack(yv, jv, lv):
            return FwdLaplArray(yv.contiguous(), FwdJacobian(jv.transpose(0, 1).contiguous(), None), lv.contiguous())

        return _tree_map(pack, y, Jy, lap)

    new_fn.__name__ = f'fwd_laplacian_{label}'
    return new_fn


def warp_without_fwd_laplacian(fn: Callable):
    """folx/wrapper.py:141-154 (the reference's spelling): a rule that drops the derivatives of its
    arguments and calls ``fn`` on the values, one walker at a time.  For functions whose result
    carries no derivative (comparisons, rounding, index computations)."""

    def wrapped(args, kwargs, sparsity_threshold: int):
        from torch.func import vmap

        args = tuple(_force(a) for a in args)
        pos = [i for i, a in enumerate(args) if _is(a) or isinstance(a, BatchedArray)]
        if not pos:
            return fn(*args, **kwargs)
        vals = tuple(args[i].x if _is(args[i]) else args[i].data for i in pos)

        def call(vs):
            full = list(args)
            for i, v in zip(pos, vs):
                full[i] = v
            return fn(*full, **kwargs)

        return _tree_map(BatchedArray, vmap(call)(vals))

    return wrapped


def wrap_elementwise(fn: Callable):
    """folx/wrapper.py:157-176: ``fn`` is applied to the value, to the Jacobian rows and to the
    Laplacian as they are (a linear map that acts on every element alone, e.g. a change of
    sign or of units); the sparsity pattern is kept."""

    def wrapped(args, kwargs, sparsity_threshold: int):
        assert len(args) == 1
        (x,) = (_force(args[0]),)
        if _is(x):
            return FwdLaplArray(fn(x.x), FwdJacobian(fn(x.jacobian.data), x.jacobian.x0_idx), fn(x.laplacian))
        if isinstance(x, BatchedArray):
            return BatchedArray(fn(x.data))
        return fn(x)

    return wrapped

"""Rule registry and the forward-Laplacian rules, each one a launch (or a few) of the HIP
kernel library.

Mirrors folx/wrapped_functions.py: ``_LAPLACE_FN_REGISTRY`` (:355-561) keyed by primitive
name, ``register_function`` / ``deregister_function`` / ``is_registered`` /
``get_laplacian`` (:564-618).  A rule has the reference's signature
``rule(args, kwargs, sparsity_threshold) -> FwdLaplArray | tuple`` (folx/api.py:444-450).
Keys are the jax primitive / jitted-function names the reference registers under
(``'dot_general'``, ``'tanh'``, ``'reduce_sum'``, ``'slogdet'``,
``'_multi_head_self_attention'`` ...), so a rule written for folx's registry plugs in
under the same name.

Unlike the reference there is no generic autodiff fallback: a primitive without a kernel
rule raises ``KeyError`` in ``get_laplacian``.
"""

from __future__ import annotations

import logging
from typing import Any, Callable

import numpy as np
import torch

from . import index_algebra as ia
from . import kernels as K
from . import sparse_ops as so
from .api import BatchedArray, FwdJacobian, FwdLaplArray

ForwardLaplacian = Callable[[tuple, dict, int], Any]

_LAPLACE_FN_REGISTRY: dict[Any, ForwardLaplacian] = {}


def register_function(primitive_or_name, laplacian: ForwardLaplacian):
    """Register a rule under a primitive / function name (folx/wrapped_functions.py:564)."""
    _LAPLACE_FN_REGISTRY[primitive_or_name] = laplacian


def deregister_function(primitive_or_name):
    del _LAPLACE_FN_REGISTRY[primitive_or_name]


def is_registered(primitive_or_name) -> bool:
    return primitive_or_name in _LAPLACE_FN_REGISTRY


def get_laplacian(primitive_or_name, wrap_if_missing: bool = False) -> ForwardLaplacian | None:
    """folx/wrapped_functions.py:597-618.  Keys are the reference's primitive / function names, or
    a callable.  ``wrap_if_missing``: a callable without a rule of its own (a torch function of
    per-walker tensors) gets the generic rule of ``folx_amd.wrapper.wrap_forward_laplacian``,
    as the reference wraps an unknown primitive; a bare name has nothing to differentiate and
    raises."""
    if primitive_or_name in _LAPLACE_FN_REGISTRY:
        return _LAPLACE_FN_REGISTRY[primitive_or_name]
    if wrap_if_missing:
        if callable(primitive_or_name):
            from .wrapper import wrap_forward_laplacian

            return wrap_forward_laplacian(primitive_or_name)
        raise KeyError(
            f'{primitive_or_name!r} has no forward-Laplacian rule; register one with '
            'folx_amd.register_function'
        )
    return None


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------


def _is(a):
    return isinstance(a, FwdLaplArray)


def _logical_shape(c) -> tuple:
    if isinstance(c, (FwdLaplArray, BatchedArray)):
        return tuple(c.shape)
    if isinstance(c, torch.Tensor):
        return tuple(c.shape)
    return tuple(np.shape(c))


def _pad_logical(t: FwdLaplArray, nd: int) -> FwdLaplArray:
    """Prepend size-1 logical axes (numpy broadcasting aligns shapes on the right)."""
    ex = nd - t.ndim
    if ex <= 0:
        return t
    one = (1,) * ex
    B, k = t.B, t.jacobian.data.shape[0]
    mask = t.jacobian.x0_idx
    if mask is not None:
        mask = mask.reshape(mask.shape[0], *one, *mask.shape[1:])
    return FwdLaplArray(
        t.x.reshape(B, *one, *t.shape),
        FwdJacobian(t.jacobian.data.reshape(k, B, *one, *t.shape), mask),
        t.laplacian.reshape(B, *one, *t.shape),
    )


def _const_tensor(c, nd: int, device) -> torch.Tensor:
    """Constant as a device tensor of shape (B or 1, *logical padded to nd dims)."""
    if isinstance(c, BatchedArray):
        d = c.data
        return d.reshape(d.shape[0], *((1,) * (nd - c.ndim)), *c.shape).contiguous()
    t = so.device_const(c, device)
    return t.reshape(1, *((1,) * (nd - t.dim())), *t.shape)


def _empty_jac(like: torch.Tensor) -> torch.Tensor:
    return torch.empty((0, *like.shape), device=like.device, dtype=torch.float32)


def _values_binary(op: str, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Binary op on derivative-free device arrays (the P = 0 case of the binary kernel)."""
    a, b = a.contiguous(), b.contiguous()
    y, _, _ = K.binary(op, a, _empty_jac(a), a, b, _empty_jac(b), b)
    return y


def _values_unary(name: str, a: torch.Tensor, param=0.0) -> torch.Tensor:
    a = a.contiguous()
    y, _, _ = K.elementwise(name, a, _empty_jac(a), a, param)
    return y


def _bmask(mask, k, out_shape):
    return None if mask is None else np.broadcast_to(mask, (k, *out_shape))


# --------------------------------------------------------------------------------------
# unary elementwise rules (kernel family 2)
# --------------------------------------------------------------------------------------

_NP_UNARY = {
    'tanh': np.tanh, 'exp': np.exp, 'log': np.log, 'sqrt': np.sqrt, 'square': np.square,
    'sin': np.sin, 'cos': np.cos, 'abs': np.abs, 'log1p': np.log1p, 'expm1': np.expm1,
    'rsqrt': lambda x: 1 / np.sqrt(x), 'reciprocal': lambda x: 1 / x,
    'logistic': lambda x: 1 / (1 + np.exp(-x)), 'silu': lambda x: x / (1 + np.exp(-x)),
    'softplus': lambda x: np.logaddexp(x, 0), 'neg': np.negative,
    'sinh': np.sinh, 'cosh': np.cosh, 'tan': np.tan, 'asin': np.arcsin, 'acos': np.arccos, 'atan': np.arctan,
    'asinh': np.arcsinh, 'acosh': np.arccosh, 'atanh': np.arctanh, 'cbrt': np.cbrt,
}


def _unary_rule(name: str) -> ForwardLaplacian:
    """``wrap_forward_laplacian(f, in_axes=())`` for a scalar function
    (folx/wrapped_functions.py:400-415): one fused pass ``y = f(x)``, ``J_y = f'(x) J``,
    ``lap_y = f'(x) lap + f''(x) sum_p J_p^2`` for dense and sparse storage alike
    (folx/jvp.py:687-697, :262-272; folx/hessian.py:87-112, gate :460-470)."""

    def rule(args, kwargs, sparsity_threshold):
        (a,) = args
        param = kwargs.get('y', kwargs.get('param', 0.0))
        if isinstance(a, BatchedArray):
            return BatchedArray(_values_unary(name, a.data, param))
        if not _is(a):
            if name == 'integer_pow':
                return np.asarray(a) ** int(param)
            if name == 'pow':
                return np.asarray(a) ** float(param)
            if name in ('erf', 'erfc', 'erf_inv', 'lgamma', 'digamma'):
                import scipy.special as sp

                return {'erf': sp.erf, 'erfc': sp.erfc, 'erf_inv': sp.erfinv, 'lgamma': sp.gammaln,
                        'digamma': sp.digamma}[name](np.asarray(a))
            return _NP_UNARY[name](np.asarray(a))
        mask = a.jacobian.x0_idx
        x, J, lap = a.x, a.jacobian.data, a.laplacian
        if mask is not None and ia.has_duplicates(mask):
            # An index listed twice at one position breaks sum_k J_k^2 = |grad|^2, so the
            # reference leaves its fast path (folx/hessian.py:460-470): the Jacobian rows
            # keep their layout (folx/jvp.py:262-272) while the Hessian term is taken on
            # the per-position unique frame (folx/hessian.py:288-340).
            y, Jy, _ = K.elementwise(name, x, J, lap, param)
            frame, _ = ia.find_out_idx([mask], [list(a.shape)], [()], False, sparsity_threshold)
            frame = frame.reshape(frame.shape[0], *a.shape)
            Jm = so.materialize(J, ia.get_index_mask(mask, frame), frame.shape[0])
            _, _, lapy = K.elementwise(name, x, Jm, lap, param)
            return FwdLaplArray(y, FwdJacobian(Jy, mask), lapy)
        y, Jy, lapy = K.elementwise(name, x, J, lap, param)
        return FwdLaplArray(y, FwdJacobian(Jy, mask), lapy)

    rule.__name__ = name
    return rule


def neg_rule(args, kwargs, sparsity_threshold):
    """``lax.neg`` is LINEAR (folx/wrapped_functions.py:361-363)."""
    (a,) = args
    if isinstance(a, BatchedArray):
        return BatchedArray(_scale_rows(a.data, 1, -1.0))
    if not _is(a):
        return -np.asarray(a)
    k = a.jacobian.data.shape[0]
    return FwdLaplArray(
        _scale_rows(a.x, 1, -1.0),
        FwdJacobian(_scale_rows(a.jacobian.data, k, -1.0), a.jacobian.x0_idx),
        _scale_rows(a.laplacian, 1, -1.0),
    )


def _scale_rows(t: torch.Tensor, rows: int, alpha: float) -> torch.Tensor:
    n = t.numel() // max(rows, 1)
    if t.numel() == 0:
        return t.clone()
    out = K.rows_affine(t.contiguous(), rows, (n,), (n,), None, None, alpha, 0.0)
    return out.reshape(t.shape)


# --------------------------------------------------------------------------------------
# binary elementwise rules
# --------------------------------------------------------------------------------------


def _affine_const(t: FwdLaplArray, c, *, mul: bool, alpha: float, beta: float) -> FwdLaplArray:
    """Triplet against a constant: ``y = alpha * x (* c) (+ beta * c)``; the Jacobian rows
    and the Laplacian are scaled the same way and never shifted (LINEAR rules,
    folx/wrapped_functions.py:361-376; mul by a constant is the one-argument case of
    MULTIPLICATION, folx/hessian.py:561-570 -> zero Hessian term)."""
    scalar = isinstance(c, (int, float)) or (not isinstance(c, (BatchedArray, torch.Tensor)) and np.ndim(c) == 0)
    cshape = () if scalar else _logical_shape(c)
    nd = max(t.ndim, len(cshape))
    t = _pad_logical(t, nd)
    out_shape = tuple(np.broadcast_shapes(t.shape, cshape))
    B, k = t.B, t.jacobian.data.shape[0]
    dev = t.x.device
    if scalar:
        cval = float(c)
        ct = None
        if mul:
            a_x = a_j = alpha * cval
            d_t, b_x = None, 0.0
        else:
            a_x = a_j = alpha
            d_t = so.device_const(np.full((1,) * (nd + 1), cval, dtype=np.float32), dev)
            b_x = beta
    else:
        ct = _const_tensor(c, nd, dev)
        a_x = a_j = alpha
        d_t, b_x = (None, 0.0) if mul else (ct, beta)
        if not mul:
            ct = None
    full = (B, *out_shape)
    x = K.rows_affine(t.x, 1, (B, *t.shape), full, ct, d_t, a_x, b_x).reshape(full)
    same = out_shape == t.shape and ct is None and a_j == 1.0
    if same:
        J, lap = t.jacobian.data, t.laplacian
    else:
        J = K.rows_affine(t.jacobian.data, k, (B, *t.shape), full, ct, None, a_j, 0.0).reshape(k, *full)
        lap = K.rows_affine(t.laplacian, 1, (B, *t.shape), full, ct, None, a_j, 0.0).reshape(full)
    return FwdLaplArray(x, FwdJacobian(J, _bmask(t.jacobian.x0_idx, k, out_shape)), lap)


def _binary_const(op: str, t: FwdLaplArray, c, t_is_left: bool) -> FwdLaplArray:
    if op == 'add':
        return _affine_const(t, c, mul=False, alpha=1.0, beta=1.0)
    if op == 'sub':
        if t_is_left:
            return _affine_const(t, c, mul=False, alpha=1.0, beta=-1.0)
        return _affine_const(t, c, mul=False, alpha=-1.0, beta=1.0)
    if op == 'mul':
        return _affine_const(t, c, mul=True, alpha=1.0, beta=0.0)
    if op == 'div':
        if t_is_left:
            if isinstance(c, BatchedArray):
                rc = BatchedArray(_values_unary('reciprocal', c.data))
            elif isinstance(c, torch.Tensor):
                rc = 1.0 / c.detach().cpu().numpy().astype(np.float64)
            else:
                rc = 1.0 / np.asarray(c, dtype=np.float64)
            return _affine_const(t, rc, mul=True, alpha=1.0, beta=0.0)
        r = _LAPLACE_FN_REGISTRY['reciprocal']((t,), {}, 0)
        return _affine_const(r, c, mul=True, alpha=1.0, beta=0.0)
    if op in ('min', 'max'):
        return _minmax_const(op, t, c)
    raise ValueError(op)


def _selection_weights(op: str, ax: torch.Tensor, bx: torch.Tensor):
    """``min`` / ``max`` of two value arrays and the weight of the first operand in the
    result's derivatives (1 where it is selected, 1/2 at a tie, else 0): the binary kernel
    applied to a Jacobian row of ones against a row of zeros."""
    shape = torch.broadcast_shapes(ax.shape, bx.shape)
    one = torch.empty((1, *ax.shape), device=ax.device, dtype=torch.float32).fill_(1.0)
    zero = so.zeros((1, *bx.shape), ax.device)
    y, w, _ = K.binary(op, ax.contiguous(), one, ax.contiguous(), bx.contiguous(), zero, bx.contiguous())
    return y, w.reshape(shape)


def _minmax_const(op: str, t: FwdLaplArray, c) -> FwdLaplArray:
    """``min`` / ``max`` against a constant: where the constant wins the derivatives vanish;
    the mask is unchanged."""
    cshape = _logical_shape(c)
    nd = max(t.ndim, len(cshape))
    t = _pad_logical(t, nd)
    out_shape = tuple(np.broadcast_shapes(t.shape, cshape))
    B, k, dev = t.B, t.jacobian.data.shape[0], t.x.device
    ct = _const_tensor(c, nd, dev)
    full = (B, *out_shape)
    y, w = _selection_weights(op, t.x, ct)
    J = K.rows_affine(t.jacobian.data, k, (B, *t.shape), full, w, None, 1.0, 0.0).reshape(k, *full)
    lap = K.rows_affine(t.laplacian, 1, (B, *t.shape), full, w, None, 1.0, 0.0).reshape(full)
    return FwdLaplArray(y.reshape(full), FwdJacobian(J, _bmask(t.jacobian.x0_idx, k, out_shape)), lap)


def _expand_rows(J: torch.Tensor, k: int, src_shape, full) -> torch.Tensor:
    """Materialise the broadcast of Jacobian rows (k, *src_shape) to (k, *full)."""
    if tuple(src_shape) == tuple(full):
        return J
    return K.rows_affine(J, k, tuple(src_shape), tuple(full), None, None, 1.0, 0.0).reshape(k, *full)


def _binary_both(op: str, a: FwdLaplArray, b: FwdLaplArray, thr: int) -> FwdLaplArray:
    nd = max(a.ndim, b.ndim)
    a, b = _pad_logical(a, nd), _pad_logical(b, nd)
    out_shape = tuple(np.broadcast_shapes(a.shape, b.shape))
    B = a.B

    def fused(Ja, Jb, mask):
        y, J, lap = K.binary(op, a.x, Ja, a.laplacian, b.x, Jb, b.laplacian)
        return FwdLaplArray(y, FwdJacobian(J, mask), lap)

    if op == 'mul' and a.jacobian.weak != b.jacobian.weak and tuple(a.shape) == tuple(b.shape):
        # one dense, one sparse operand of the same shape: the product takes the sparse rows
        # as they are (same result as densifying them first, which is what follows otherwise)
        dn, sp = (b, a) if a.jacobian.weak else (a, b)
        m = np.broadcast_to(sp.jacobian.x0_idx, (sp.jacobian.x0_idx.shape[0], *out_shape))
        k = m.shape[0]
        if k <= 8 and sp.jacobian.max_n < dn.jacobian.data.shape[0] and not ia.has_duplicates(m):
            table = so.device_table(np.ascontiguousarray(m.reshape(k, -1)), a.x.device)
            y, J, lap = K.mul_sparse(dn.x, dn.jacobian.data, dn.laplacian, sp.x, sp.jacobian.data, sp.laplacian,
                                     table)
            return FwdLaplArray(y, FwdJacobian(J, None), lap)
    if not (a.jacobian.weak and b.jacobian.weak):
        # Any dense operand: the reference adds the per-operand results through
        # FwdJacobian.__add__, which densifies (folx/jvp.py:742-796, folx/api.py:233-236).
        Ja, Jb = a.jacobian.dense_array, b.jacobian.dense_array
        P = max(Ja.shape[0], Jb.shape[0])
        return fused(so.pad_rows(Ja, P), so.pad_rows(Jb, P), None)

    ma = np.broadcast_to(a.jacobian.x0_idx, (a.jacobian.x0_idx.shape[0], *out_shape))
    mb = np.broadcast_to(b.jacobian.x0_idx, (b.jacobian.x0_idx.shape[0], *out_shape))
    ka, kb = ma.shape[0], mb.shape[0]
    if ka == kb and np.array_equal(ma, mb) and not ia.has_duplicates(ma) and (
        ka == 1 or ia.rows_distinct(ma)
    ):
        # identical masks: merged rows = the rows themselves, and the intersection /
        # union frame is the mask itself, so one fused launch on k rows is the rule
        return fused(a.jacobian.data, b.jacobian.data, ma)

    # ---- general sparse case: merged one-hot rows (folx/jvp.py:273-317) -----------------
    res_mask, inv = ia.merge_rows([ma, mb])
    full = (B, *out_shape)
    if op in ('add', 'sub'):
        ca = cb = None
        sa, sb = 1.0, (1.0 if op == 'add' else -1.0)
    elif op == 'mul':
        ca, cb, sa, sb = b.x, a.x, 1.0, 1.0
    elif op in ('min', 'max'):
        # the selected operand's rows pass through (LINEAR, folx/wrapped_functions.py:508-513)
        y, ca = _selection_weights(op, a.x, b.x)
        cb = K.rows_affine(ca, 1, tuple(ca.shape), tuple(ca.shape), None,
                           so.device_const(np.ones((1,) * ca.dim(), dtype=np.float32), ca.device),
                           -1.0, 1.0).reshape(ca.shape)
        sa = sb = 1.0
    else:  # div: d/da = 1/b, d/db = -a/b^2
        rb = _values_unary('reciprocal', b.x)
        q = _values_binary('mul', a.x, rb)
        ca, cb, sa, sb = rb, _values_binary('mul', q, rb), 1.0, -1.0

    def scaled_row(J, r, src_shape, c, alpha):
        row = J[r : r + 1].contiguous()
        return K.rows_affine(row, 1, (B, *src_shape), full, c, None, alpha, 0.0).reshape(1, *full)

    rows = [scaled_row(a.jacobian.data, r, a.shape, ca, sa) for r in range(ka)]
    rows += [scaled_row(b.jacobian.data, r, b.shape, cb, sb) for r in range(kb)]
    merged = []
    for o in range(res_mask.shape[0]):
        members = np.nonzero(inv == o)[0]
        acc = rows[members[0]]
        for m in members[1:]:
            acc = so.add_rowstacks(acc, rows[m])
        merged.append(acc)
    J_out = torch.cat(merged, dim=0) if len(merged) > 1 else merged[0]

    if op in ('add', 'sub'):
        y = K.rows_affine(a.x, 1, (B, *a.shape), full, None,
                          _expand_rows(b.x, 1, (B, *b.shape), full).reshape(full), 1.0, sb).reshape(full)
        lap = K.rows_affine(a.laplacian, 1, (B, *a.shape), full, None,
                            _expand_rows(b.laplacian, 1, (B, *b.shape), full).reshape(full), 1.0, sb).reshape(full)
        return FwdLaplArray(y, FwdJacobian(J_out, res_mask), lap)
    if op in ('min', 'max'):
        _, _, lap = K.binary(op, a.x, _empty_jac(a.x), a.laplacian, b.x, _empty_jac(b.x), b.laplacian)
        return FwdLaplArray(y.reshape(full), FwdJacobian(J_out, res_mask), lap.reshape(full))

    # Hessian term on the static index frame (folx/hessian.py:288-340, :379-428):
    # intersection for mul (LINEAR_IN_ONE), union for div; dense when the frame says so.
    frame, dense_out = ia.find_out_idx(
        [ma, mb], [list(out_shape), list(out_shape)], [(), ()], op == 'mul', thr
    )
    if dense_out:
        Ja, Jb = a.jacobian.dense_array, b.jacobian.dense_array
        P = max(Ja.shape[0], Jb.shape[0])
        Ja, Jb = so.pad_rows(Ja, P), so.pad_rows(Jb, P)
    else:
        frame = frame.reshape(frame.shape[0], *out_shape)
        M = frame.shape[0]
        Ja = so.materialize(_expand_rows(a.jacobian.data, ka, (B, *a.shape), full), ia.get_index_mask(ma, frame), M)
        Jb = so.materialize(_expand_rows(b.jacobian.data, kb, (B, *b.shape), full), ia.get_index_mask(mb, frame), M)
    if Ja.shape[0] == 0:
        Ja = Jb = _empty_jac(a.x.expand(full))
    y, _, lap = K.binary(op, a.x, Ja, a.laplacian, b.x, Jb, b.laplacian)
    return FwdLaplArray(y, FwdJacobian(J_out, res_mask), lap)


_NP_BINARY = {'add': np.add, 'sub': np.subtract, 'mul': np.multiply, 'div': np.divide,
              'min': np.minimum, 'max': np.maximum}


def _binary_rule(op: str) -> ForwardLaplacian:
    def rule(args, kwargs, sparsity_threshold):
        a, b = args
        if _is(a) and _is(b):
            return _binary_both(op, a, b, sparsity_threshold)
        if _is(a):
            return _binary_const(op, a, b, True)
        if _is(b):
            return _binary_const(op, b, a, False)
        if isinstance(a, BatchedArray) or isinstance(b, BatchedArray):
            ref = a if isinstance(a, BatchedArray) else b
            nd = max(len(_logical_shape(a)), len(_logical_shape(b)))
            ta = _const_tensor(a, nd, ref.data.device)
            tb = _const_tensor(b, nd, ref.data.device)
            Bn = ref.B
            ta = ta.expand(Bn, *ta.shape[1:]) if ta.shape[0] == 1 else ta
            tb = tb.expand(Bn, *tb.shape[1:]) if tb.shape[0] == 1 else tb
            return BatchedArray(_values_binary(op, ta.contiguous(), tb.contiguous()))
        return _NP_BINARY[op](np.asarray(a), np.asarray(b))

    rule.__name__ = op
    return rule


# --------------------------------------------------------------------------------------
# dense layer (kernel family 1)
# --------------------------------------------------------------------------------------


def dot_general(args, kwargs, sparsity_threshold: int = 0):
    """``h @ W`` with exactly one operand carrying derivatives and the last axis of ``h``
    contracted with the first axis of a constant matrix ``W (K, N)``
    (``_dot_general_one_constant``, folx/wrapped_functions.py:71-171): the product is
    applied to x, to every Jacobian row and to the Laplacian in one GEMM launch.
    ``kwargs['bias']`` (constant, shape (N,)) is added to x only.  ``kwargs['residual']``
    (a triplet of the output shape) is added to the result; with matching dense Jacobians
    the addition happens in the GEMM epilogue, otherwise through the ``add`` rule.

    Sparse ``h``: rows pass through when the mask is constant along the contracted axis;
    otherwise they are first aligned to the per-position union frame over that axis
    (:113-130); a union wider than the threshold falls back to the dense Jacobian, which
    is what the reference's general path produces for this case (folx/jvp.py:224-230).
    """
    h, W = args
    if kwargs.get('batched_const'):
        return _dot_batched_const(h, W, sparsity_threshold)
    if isinstance(h, LazyConcat):
        return _dot_parts(h, W, kwargs, sparsity_threshold)
    bias = kwargs.get('bias')
    residual = kwargs.get('residual')
    row_slice = kwargs.get('row_slice')
    if kwargs.get('act') is not None or kwargs.get('norm') is not None:
        return _dot_then_act(h, W, dict(kwargs), sparsity_threshold)
    if row_slice is not None:
        # the slice is consumed in place by the kernel when the Jacobian needs no re-indexing;
        # otherwise it is an ordinary ``slice`` in front of the product
        lo, hi = row_slice
        plain_rows = _is(h) and not _is(W) and h.ndim >= 2 and (
            h.jacobian.x0_idx is None or not ia.dot_projection(h.jacobian.x0_idx, -1, sparsity_threshold)[1])
        if not plain_rows:
            hs = getitem_rule((h,), {'idx': (Ellipsis, slice(lo, hi), slice(None))}, sparsity_threshold)
            return dot_general((hs, W), {'bias': bias, 'residual': residual}, sparsity_threshold)
    if not _is(h):
        if _is(W):
            raise NotImplementedError('dot_general: constant @ triplet is not supported; transpose the product')
        if isinstance(h, BatchedArray):
            raise NotImplementedError('dot_general on walker-varying constants')
        y = np.asarray(h) @ np.asarray(W)
        return y if bias is None else y + np.asarray(bias)
    if _is(W):
        out = _dot_two_operands(h, W, sparsity_threshold)
        if bias is not None:
            out = _LAPLACE_FN_REGISTRY['add']((out, bias), {}, sparsity_threshold)
        if residual is not None:
            out = _LAPLACE_FN_REGISTRY['add']((residual, out), {}, sparsity_threshold)
        return out
    dev = h.x.device
    Wt = so.device_const(W, dev)
    bt = None if bias is None else so.device_const(bias, dev)
    Kd, N = Wt.shape
    assert h.shape[-1] == Kd, f'dot: contracting {h.shape} with {tuple(Wt.shape)}'
    J, mask = h.jacobian.data, h.jacobian.x0_idx
    out_lead = tuple(h.shape[:-1])
    if row_slice is not None:
        out_lead = (*out_lead[:-1], row_slice[1] - row_slice[0])
        if mask is not None:
            mask = np.broadcast_to(mask, (mask.shape[0], *h.shape))[..., row_slice[0]:row_slice[1], :]
    new_mask = None
    if mask is not None:
        proj, aligned = ia.dot_projection(mask, -1, sparsity_threshold)
        if proj is None:
            logging.info('dot_general: union over the contracted axis exceeds the sparsity threshold; densifying')
            J = h.jacobian.dense_array
        else:
            if aligned:
                J = so.materialize(J, ia.get_index_mask(mask, proj), proj.shape[0])
            new_mask = np.broadcast_to(proj, (proj.shape[0], *out_lead, N))
    res = None
    if residual is not None and _is(residual):
        rj = residual.jacobian
        if (
            new_mask is None and not rj.weak and rj.data.shape[0] == J.shape[0]
            and tuple(residual.shape) == (*out_lead, N)
        ):
            res, residual = (residual.x, rj.data, residual.laplacian), None
    y, Jy, lapy = K.dense(h.x, J, h.laplacian, Wt, bt, res, row_slice)
    if (
        residual is not None and _is(residual) and new_mask is None and residual.jacobian.weak
        and tuple(residual.shape) == (*out_lead, N) and residual.jacobian.max_n < Jy.shape[0]
    ):
        # sparse skip connection into a dense result: the GEMM output is fresh and owned
        # here, so the few stored rows are added into it in place instead of being
        # materialised to P rows first
        so.add_sparse_rows_(Jy, residual.jacobian.data, residual.jacobian.x0_idx)
        y = so.add_rowstacks(y, residual.x)
        lapy = so.add_rowstacks(lapy, residual.laplacian)
        residual = None
    out = FwdLaplArray(y, FwdJacobian(Jy, new_mask), lapy)
    if residual is not None:
        out = _LAPLACE_FN_REGISTRY['add']((residual, out), {}, sparsity_threshold)
    return out


def _dot_batched_const(h: FwdLaplArray, W, thr: int) -> FwdLaplArray:
    """``h (Bt, I, Kc) x W (Bt, Kc, J) -> (Bt, I, J)`` per walker, ``W`` a constant with a batch axis
    (per-head weights): the case of ``_dot_general_one_constant`` in which the constant operand has
    batch dimensions (folx/wrapped_functions.py:71-171; the front end has brought any dimension
    numbers to this form).  Linear in ``h``: the product is applied to x, to every Jacobian row
    and to the Laplacian (:167-169) by one launch of the batched product kernel, which reads the
    constant once per batch element.  Sparse rows pass through when their mask is constant along
    the contracted axis, are aligned to the per-position union over it otherwise, and a union
    wider than the threshold densifies (:113-157)."""
    dev = h.x.device
    Wt = so.device_const(W, dev)
    Bt, I, Kc = h.shape
    assert tuple(Wt.shape[:2]) == (Bt, Kc), f'dot_general: contracting {tuple(h.shape)} with {tuple(Wt.shape)}'
    N = Wt.shape[2]
    J, mask = h.jacobian.data, h.jacobian.x0_idx
    new_mask = None
    if mask is not None:
        mask = np.broadcast_to(mask, (mask.shape[0], Bt, I, Kc))
        proj, aligned = ia.dot_projection(mask, -1, thr)
        if proj is None:
            logging.info('dot_general: union over the contracted axis exceeds the sparsity threshold; densifying')
            J = h.jacobian.dense_array
        else:
            if aligned:
                J = so.materialize(J, ia.get_index_mask(mask, proj), proj.shape[0])
            new_mask = np.broadcast_to(proj, (proj.shape[0], Bt, I, N))
    y, Jy, lapy = K.dot_const(h.x, J, h.laplacian, Wt)
    return FwdLaplArray(y, FwdJacobian(Jy, new_mask), lapy)


def _zero_rows_below(W, k_pad: int):
    """``W`` with ``k_pad`` zero rows appended (the partner of zero feature columns appended to the input)."""
    if isinstance(W, torch.Tensor):  # a caller-owned device tensor: padded on every call (it may change in place)
        return torch.cat([W.to(torch.float32), W.new_zeros((k_pad, W.shape[1]), dtype=torch.float32)], dim=0)
    return np.concatenate([np.asarray(W, dtype=np.float32), np.zeros((k_pad, np.shape(W)[1]), dtype=np.float32)], axis=0)


def _dot_then_act(h, W, kwargs, thr: int):
    """``residual + act(layer_norm(h) @ W + bias)`` with ``act`` and ``layer_norm`` optional.
    A Dense + activation layer is ONE rule when the fused kernels take its shape
    (``kernels.dense_act_supported``) and the result's Jacobian rows are plain (dense, or
    sparse without an index listed twice at a position, where sum_k J_k^2 is the Hessian
    term, folx/hessian.py:460-470); LayerNorm joins the same rule for dense Jacobians and
    wide layers (``kernels.norm_dense_supported``).  Otherwise the ``layer_norm`` rule, the
    ``dot_general`` rule and the elementwise rule one after the other, which is also what
    defines the result."""
    act = kwargs.pop('act', None)
    param = kwargs.pop('act_param', 0.0)
    residual = kwargs.pop('residual', None)
    norm = kwargs.pop('norm', None)
    bias = kwargs.get('bias')
    if norm is not None:
        gamma, beta, eps = (norm.gamma, norm.beta, norm.eps) if isinstance(norm, LazyLayerNorm) else norm
        if (
            _is(h) and not _is(W) and kwargs.get('row_slice') is None and np.ndim(W) == 2
            and h.jacobian.x0_idx is None
            and K.norm_dense_supported(act, *np.shape(W), rows=h.x.numel() // max(h.x.shape[-1], 1),
                                       P=h.jacobian.data.shape[0])
        ):
            dev = h.x.device
            g = None if gamma is None else so.device_const(gamma, dev)
            b = None if beta is None else so.device_const(beta, dev)
            bt = None if bias is None else so.device_const(bias, dev)
            y, Jy, lapy = K.norm_dense(act, h.x, h.jacobian.data, h.laplacian, g, b, float(eps),
                                       so.device_const(W, dev), bt, param)
            out = FwdLaplArray(y, FwdJacobian(Jy, None), lapy)
            if residual is not None:
                out = _LAPLACE_FN_REGISTRY['add']((residual, out), {}, thr)
            return out
        if isinstance(norm, LazyLayerNorm):
            h = norm.value(thr)
        else:
            h = layer_norm_rule((h, gamma, beta), {'eps': eps}, thr)
    if act is None:
        return dot_general((h, W), {**kwargs, 'residual': residual}, thr)
    k_pad = 0
    if (_is(h) and not _is(W) and kwargs.get('row_slice') is None and np.ndim(W) == 2
            and np.shape(W)[1] > 128 and np.shape(W)[0] % 16 != 0 and np.shape(W)[0] >= 16):
        # a wide layer whose input width is no multiple of 16 (a first layer fed by raw features): the fused
        # kernel takes it with the feature axis padded by zero columns against zero rows of W, which costs one
        # copy of the input triplet and saves the pre-activation triplet's trip through memory
        k_pad = -np.shape(W)[0] % 16
        W = _zero_rows_below(W, k_pad)
    K_in = np.shape(W)[0] - k_pad
    fused = (
        _is(h) and not _is(W) and kwargs.get('row_slice') is None and np.ndim(W) == 2
        and K.dense_act_supported(act, *np.shape(W), rows=h.x.numel() // max(h.x.shape[-1], 1))
    )
    J = new_mask = None
    if fused:
        J, mask = h.jacobian.data, h.jacobian.x0_idx
        N = np.shape(W)[1]
        if mask is not None:
            proj, aligned = ia.dot_projection(mask, -1, thr)
            if proj is None:
                J = h.jacobian.dense_array
            elif ia.has_duplicates(proj):
                fused = False
            else:
                if aligned:
                    J = so.materialize(J, ia.get_index_mask(mask, proj), proj.shape[0])
                new_mask = np.broadcast_to(proj, (proj.shape[0], *h.shape[:-1], N))
    if fused:  # the number of Jacobian rows decides whether the wide kernel's tiles are well filled
        fused = K.dense_act_supported(act, *np.shape(W), rows=h.x.numel() // max(h.x.shape[-1], 1), P=J.shape[0])
    if not fused and k_pad:
        W = W[:K_in]
    if fused:
        dev = h.x.device
        Wt = so.device_const(W, dev)
        bt = None if bias is None else so.device_const(bias, dev)
        res = None
        hx, hl = h.x, h.laplacian
        if k_pad:
            padk = lambda t: torch.nn.functional.pad(t, (0, k_pad))
            hx, J, hl = padk(hx), padk(J), padk(hl)
        if (_is(residual) and K.dense_act_residual_supported(*np.shape(W))
                and tuple(residual.shape) == (*h.shape[:-1], np.shape(W)[1])
                and residual.jacobian.data.shape[0] == J.shape[0]):
            # a skip connection on the same row frame (both dense, or the same sparse mask) is added in
            # the kernel's epilogue (the add rule would take the identical-masks branch, _binary_both)
            rm = residual.jacobian.x0_idx
            same = (rm is None and new_mask is None) or (
                rm is not None and new_mask is not None
                and np.array_equal(np.broadcast_to(rm, (rm.shape[0], *residual.shape)), new_mask)
                and not ia.has_duplicates(new_mask) and (new_mask.shape[0] == 1 or ia.rows_distinct(new_mask)))
            if same:
                res = (residual.x.contiguous(), residual.jacobian.data.contiguous(), residual.laplacian.contiguous())
                residual = None
        y, Jy, lapy = K.dense_act(act, hx, J, hl, Wt, bt, param, res)
        out = FwdLaplArray(y, FwdJacobian(Jy, new_mask), lapy)
    else:
        out = dot_general((h, W), kwargs, thr)
        out = _LAPLACE_FN_REGISTRY[act]((out,), {'param': param}, thr)
    if residual is not None:
        out = _LAPLACE_FN_REGISTRY['add']((residual, out), {}, thr)
    return out


def _dot_two_operands(lhs: FwdLaplArray, rhs: FwdLaplArray, thr: int) -> FwdLaplArray:
    """Matrix product of two derivative-carrying operands with ``numpy.matmul`` shapes,
    ``lhs (..., i, k) @ rhs (..., k, j)`` (1-D operands as in matmul).

    Dense Jacobians (or sparse ones for which the reference takes its general path): ONE rule,
    ``kernels.dot_two`` -- JVP both ways plus the DOT_PRODUCT Hessian term 2 tr(J_l J_r^T)
    (folx/wrapped_functions.py:294-309, folx/hessian.py:177-188) as batched matrix products;
    the (..., i, j, k) intermediate is never formed.

    Both operands sparse and the product's sparse Jacobian cheaper than the dense ones (the cost
    gate of folx/wrapped_functions.py:253-262): the reference's ``rearrange`` + ``mul_sum``
    decomposition (:47-68, :263-286) through the ``mul`` and ``reduce_sum`` rules, which keeps
    the result sparse."""
    a_vec, b_vec = lhs.ndim == 1, rhs.ndim == 1
    la = (1, lhs.shape[0]) if a_vec else tuple(lhs.shape)
    rb = (rhs.shape[0], 1) if b_vec else tuple(rhs.shape)
    assert la[-1] == rb[-2], f'matmul: contracting {tuple(lhs.shape)} with {tuple(rhs.shape)}'
    same_batch = la[:-2] == rb[:-2]
    use_mul_sum = not same_batch or la[-1] > K.DOT_TWO_KMAX
    if same_batch and lhs.jacobian.weak and rhs.jacobian.weak:
        inter = int(np.prod((*la, rb[-1]), dtype=np.int64))
        in_size = max(int(np.prod(la, dtype=np.int64)), int(np.prod(rb, dtype=np.int64)))
        k_mul = lhs.jacobian.data.shape[0] + rhs.jacobian.data.shape[0]
        n_dense = max(lhs.jacobian.max_n, rhs.jacobian.max_n) + 1
        use_mul_sum = use_mul_sum or inter == in_size or k_mul * inter < n_dense * in_size
    if use_mul_sum:
        return _dot_mul_sum(lhs, rhs, a_vec, b_vec)
    Ja, Jb = lhs.jacobian.dense_array, rhs.jacobian.dense_array
    P = max(Ja.shape[0], Jb.shape[0])
    Ja, Jb = so.pad_rows(Ja, P), so.pad_rows(Jb, P)
    B = lhs.B
    NB0 = B * int(np.prod(la[:-2], dtype=np.int64))
    va = lambda t, lead: t.reshape(*lead, NB0, 1, la[-2], la[-1])
    vb = lambda t, lead: t.reshape(*lead, NB0, 1, rb[-2], rb[-1])
    y, Jy, lapy = K.dot_two(va(lhs.x.contiguous(), ()), va(Ja.contiguous(), (P,)), va(lhs.laplacian.contiguous(), ()),
                            vb(rhs.x.contiguous(), ()), vb(Jb.contiguous(), (P,)), vb(rhs.laplacian.contiguous(), ()))
    out_shape = (*la[:-2], *(() if a_vec else (la[-2],)), *(() if b_vec else (rb[-1],)))
    return FwdLaplArray(y.reshape(B, *out_shape), FwdJacobian(Jy.reshape(P, B, *out_shape), None),
                        lapy.reshape(B, *out_shape))


def _dot_mul_sum(lhs: FwdLaplArray, rhs: FwdLaplArray, a_vec: bool, b_vec: bool) -> FwdLaplArray:
    """Both operands are rearranged so that the contracted axis is last and broadcast against
    each other, then multiplied and summed (folx/wrapped_functions.py:47-68, :263-286)."""
    from . import numpy as fnp

    a, b = lhs, rhs
    if a_vec:
        a = fnp.expand_dims(a, 0)
    if b_vec:
        b = fnp.expand_dims(b, 1)
    bt = fnp.swapaxes(b, -1, -2)  # (..., j, k)
    prod = fnp.multiply(fnp.expand_dims(a, -2), fnp.expand_dims(bt, -3))  # (..., i, j, k)
    out = fnp.sum(prod, axis=-1)
    if b_vec:
        out = fnp.squeeze(out, -1)
    if a_vec:
        out = fnp.squeeze(out, -1 if b_vec else -2)
    return out


class Deferred:
    """The result of a rule that has not been evaluated yet.

    The reference sees a whole jaxpr before anything runs and XLA fuses the emitted operations
    afterwards; a define-by-run front end sees one call at a time.  The functions of
    ``folx_amd.numpy`` therefore return a handle of this kind where a later call may be able to
    take the operation into its own rule (LayerNorm into the product that consumes it, an
    activation and a skip connection into the product in front of them, a slice into the
    product or the sum that reads it, a concatenation into the product, an elementwise factor
    and a transposition into ``slogdet``).  A consumer that knows the handle absorbs it; every
    other use -- any rule, an attribute such as ``.x`` or ``.jacobian``, the end of
    ``forward_laplacian`` -- evaluates it through the ordinary rule, once (``value``).  Either
    way the triplet is the one the ordinary rules define."""

    __slots__ = ('_value', 'thr')
    __array_ufunc__ = None   # `array <op> handle` goes to the reflected methods

    def __init__(self, thr: int):
        self._value, self.thr = None, int(thr)

    def _evaluate(self) -> FwdLaplArray:
        raise NotImplementedError

    def value(self, sparsity_threshold=None) -> FwdLaplArray:
        if self._value is None:
            from . import numpy as fnp

            with fnp.sparsity_threshold(self.thr if sparsity_threshold is None else sparsity_threshold):
                self._value = self._evaluate()
        return self._value

    # the surface of a FwdLaplArray -----------------------------------------------------------------
    @property
    def ndim(self):
        return len(self.shape)

    @property
    def size(self):
        return int(np.prod(self.shape, dtype=int))

    x = property(lambda self: self.value().x)
    jacobian = property(lambda self: self.value().jacobian)
    laplacian = property(lambda self: self.value().laplacian)
    B = property(lambda self: self.value().B)
    dtype = property(lambda self: torch.float32)
    dense_jacobian = property(lambda self: self.value().jacobian.dense_array)

    def __iter__(self):
        return iter(self.value())

    def __repr__(self):
        return f'{type(self).__name__}(shape={self.shape}, evaluated={self._value is not None})'


for _name in ('__add__', '__radd__', '__sub__', '__rsub__', '__mul__', '__rmul__', '__truediv__', '__rtruediv__',
              '__neg__', '__matmul__', '__getitem__', 'reshape', 'sum', '__rmatmul__', '__pow__', '__rpow__', '__abs__',
              '__gt__', '__ge__', '__lt__', '__le__', 'T', 'transpose', 'swapaxes', 'mean'):
    setattr(Deferred, _name, getattr(FwdLaplArray, _name))  # the same sugar: everything goes through folx_amd.numpy


def force(v):
    """``v`` with every deferred value (also inside a tuple or list) replaced by its triplet."""
    if isinstance(v, Deferred):
        return v.value()
    if isinstance(v, (tuple, list)) and any(isinstance(t, Deferred) for t in v):
        return type(v)(force(t) for t in v)
    return v


class LazyLayerNorm(Deferred):
    """``layer_norm(h, gamma, beta, eps)``: a product that can take LayerNorm into its own rule
    reads ``h`` directly, any other consumer evaluates the ``layer_norm`` rule -- once, however
    many ask."""

    __slots__ = ('h', 'gamma', 'beta', 'eps')

    def __init__(self, h, gamma, beta, eps, thr=0):
        super().__init__(thr)
        self.h, self.gamma, self.beta, self.eps = h, gamma, beta, float(eps)

    shape = property(lambda self: tuple(self.h.shape))

    def _evaluate(self):
        return layer_norm_rule((self.h, self.gamma, self.beta), {'eps': self.eps}, self.thr)


class LazyBroadcast(Deferred):
    """``broadcast_to(a, shape)``; a concatenation that a product reads in parts takes it as it is."""

    __slots__ = ('a', 'shape')

    def __init__(self, a, shape, thr=0):
        super().__init__(thr)
        self.a, self.shape = a, tuple(shape)

    def _evaluate(self):
        off = len(self.shape) - self.a.ndim
        return _LAPLACE_FN_REGISTRY['broadcast_in_dim'](
            (self.a,), {'shape': self.shape, 'broadcast_dimensions': tuple(range(off, len(self.shape)))}, self.thr)


class LazyConcat(Deferred):
    """``concatenate(parts, axis=-1)``: a product that can read its operand in parts never forms
    the concatenation (nor the broadcasts among the parts)."""

    __slots__ = ('parts',)

    def __init__(self, parts, thr=0):
        super().__init__(thr)
        self.parts = tuple(parts)

    @property
    def shape(self):
        lead = tuple(self.parts[0].shape[:-1])
        return (*lead, int(np.sum([t.shape[-1] for t in self.parts])))

    def _evaluate(self):
        return concatenate_rule(tuple(force(t) for t in self.parts), {'dimension': -1}, self.thr)


class LazySlice(Deferred):
    """``a[..., lo:hi, ...]`` along ONE axis: a product reads the rows in place (axis in front of
    the feature axis), a sum over that axis reads its window in place."""

    __slots__ = ('a', 'axis', 'lo', 'hi')

    def __init__(self, a, axis, lo, hi, thr=0):
        super().__init__(thr)
        self.a, self.axis, self.lo, self.hi = a, int(axis), int(lo), int(hi)

    @property
    def shape(self):
        s = list(self.a.shape)
        s[self.axis] = self.hi - self.lo
        return tuple(s)

    def _evaluate(self):
        idx = tuple(slice(self.lo, self.hi) if i == self.axis else slice(None) for i in range(self.axis + 1))
        return getitem_rule((self.a,), {'idx': idx}, self.thr)


class LazyDot(Deferred):
    """``h @ W`` with a constant ``W`` whose epilogue is still open: a constant vector added to it
    becomes the bias, a scalar function applied to it the activation of the same rule, a triplet
    of its shape added to it the skip connection.  ``kwargs`` are those of the ``dot_general``
    rule (bias, act, norm, row_slice); evaluation is that rule."""

    __slots__ = ('h', 'W', 'kwargs', 'shape')

    def __init__(self, h, W, kwargs, shape, thr=0):
        super().__init__(thr)
        self.h, self.W, self.kwargs, self.shape = h, W, dict(kwargs), tuple(shape)

    def with_(self, **kw):
        return LazyDot(self.h, self.W, {**self.kwargs, **kw}, self.shape, self.thr)

    def _evaluate(self, residual=None):
        return dot_general((self.h, self.W), {**self.kwargs, 'residual': residual}, self.thr)

    def value_with_residual(self, residual):
        """``residual + (this product)`` as one rule; the handle itself stays unevaluated."""
        from . import numpy as fnp

        with fnp.sparsity_threshold(self.thr):
            return self._evaluate(residual)


class LazyMul(Deferred):
    """``a * b`` of two triplets of one shape; ``slogdet`` multiplies a factor while it loads its
    matrices."""

    __slots__ = ('a', 'b')

    def __init__(self, a, b, thr=0):
        super().__init__(thr)
        self.a, self.b = a, b

    shape = property(lambda self: tuple(self.a.shape))

    def _evaluate(self):
        return _LAPLACE_FN_REGISTRY['mul']((self.a, self.b), {}, self.thr)


class LazyTranspose(Deferred):
    """``transpose(a, perm)`` that moves one axis in front of the last one and keeps the order of
    the others: the layout ``slogdet`` reads in place (matrix rows on another axis)."""

    __slots__ = ('a', 'perm')

    def __init__(self, a, perm, thr=0):
        super().__init__(thr)
        self.a, self.perm = a, tuple(perm)

    shape = property(lambda self: tuple(self.a.shape[i] for i in self.perm))

    @property
    def row_axis(self):
        return self.perm[-2]

    def _evaluate(self):
        return transpose_rule((force(self.a),), {'permutation': self.perm}, self.thr)


def _dot_parts(lc: LazyConcat, W, kwargs, thr: int):
    """``act(concatenate(parts) @ W + bias)`` with the Jacobian read part by part
    (``kernels.dense_act_parts``) when every part is a triplet of the output's leading shape,
    or a per-walker vector broadcast to it, with a width that is a multiple of 16, and the
    layer is one the wide fused kernel takes; otherwise the concatenation is evaluated and
    the product goes the usual way."""
    act, param, residual = kwargs.get('act'), kwargs.get('act_param', 0.0), kwargs.get('residual')
    ok = (act is not None and kwargs.get('norm') is None and kwargs.get('row_slice') is None and not _is(W)
          and np.ndim(W) == 2 and 1 <= len(lc.parts) <= 8)
    lead = None
    if ok:
        for t in lc.parts:
            src = t.a if isinstance(t, LazyBroadcast) else t
            if not _is(src) or src.ndim < 1 or src.shape[-1] % 16 != 0:
                ok = False
                break
            if isinstance(t, LazyBroadcast):
                ok = ok and src.ndim == 1 and t.shape[-1] == src.shape[-1]
                tl = tuple(t.shape[:-1])
            else:
                tl = tuple(src.shape[:-1])
            if lead is None:
                lead = tl
            ok = ok and tl == lead
    if ok:
        first = lc.parts[0].a if isinstance(lc.parts[0], LazyBroadcast) else lc.parts[0]
        B, dev = first.B, first.x.device
        group = int(np.prod(lead, dtype=np.int64))
        Ktot = sum((t.a if isinstance(t, LazyBroadcast) else t).shape[-1] for t in lc.parts)
        srcs = [t.a if isinstance(t, LazyBroadcast) else t for t in lc.parts]
        P = max(u.jacobian.max_n + 1 if u.jacobian.weak else u.jacobian.data.shape[0] for u in srcs)
        ok = (np.shape(W)[0] == Ktot and np.shape(W)[1] > 128 and group >= 1
              and K.dense_act_supported(act, Ktot, np.shape(W)[1], rows=B * group, P=P))
    if not ok:
        kw = dict(kwargs)
        Kin = np.shape(W)[0] if np.ndim(W) == 2 else 0
        if (act is not None and kwargs.get('norm') is None and kwargs.get('row_slice') is None and not _is(W)
                and np.ndim(W) == 2 and np.shape(W)[1] > 128 and Kin % 16 != 0 and Kin >= 16 and Kin == lc.shape[-1]):
            # a wide layer over a concatenation whose width is no multiple of 16: the zero columns that the fused
            # kernel needs (see _dot_then_act) join the concatenation as one more part instead of a second copy
            k_pad = -Kin % 16
            zero = np.zeros((*lc.shape[:-1], k_pad), dtype=np.float32)
            h = concatenate_rule(tuple(force(t) for t in lc.parts) + (zero,), {'dimension': -1}, thr)
            return dot_general((h, _zero_rows_below(W, k_pad)), kw, thr)
        return dot_general((lc.value(thr), W), kw, thr)
    bias = kwargs.get('bias')
    res = None  # a skip connection with the same dense rows goes into the kernel's epilogue
    if (_is(residual) and residual.jacobian.x0_idx is None and residual.jacobian.data.shape[0] == P
            and tuple(residual.shape) == (*lead, np.shape(W)[1])):
        res = (residual.x.contiguous(), residual.jacobian.data.contiguous(), residual.laplacian.contiguous())
    Wt = so.device_const(W, dev)
    w_const = not isinstance(W, torch.Tensor)  # a numpy constant: its device copy is never written again
    bt = None if bias is None else so.device_const(bias, dev)
    is_b = [isinstance(t, LazyBroadcast) for t in lc.parts]
    wds = [u.shape[-1] for u in srcs]
    ends = np.cumsum(wds)
    ranges = [(int(e - w), int(e)) for e, w in zip(ends, wds)]
    pre = None
    if any(is_b) and not all(is_b) and group > 1:
        # The per-walker (broadcast) parts meet their rows of W ONCE per walker: a dense layer on B
        # rows whose result enters the main product in front of the activation.  The main product
        # then only contracts the per-position parts -- for a FermiNet layer 320 of 832 features.
        for u, (lo, hi) in [(u, r) for u, r, b_ in zip(srcs, ranges, is_b) if b_]:
            # one product per broadcast part, each adding the sum so far in its epilogue (no concatenation)
            pre = K.dense(u.x, so.pad_rows(u.jacobian.dense_array, P), u.laplacian, so.weight_rows(Wt, ((lo, hi),), cache=w_const), None,
                          pre)
        keep = [i for i, b_ in enumerate(is_b) if not b_]
        Wt = so.weight_rows(Wt, tuple(ranges[i] for i in keep), cache=w_const)
        parts_, srcs_ = [lc.parts[i] for i in keep], [srcs[i] for i in keep]
    else:
        parts_, srcs_ = list(lc.parts), srcs
    xs, ls, Js, widths, flags = [], [], [], [], []
    for t, u in zip(parts_, srcs_):
        J = so.pad_rows(u.jacobian.dense_array, P).contiguous()
        if isinstance(t, LazyBroadcast):
            shp = (B, *([1] * len(lead)), u.shape[-1])
            xs.append(u.x.reshape(shp).expand(B, *lead, u.shape[-1]))
            ls.append(u.laplacian.reshape(shp).expand(B, *lead, u.shape[-1]))
        else:
            xs.append(u.x), ls.append(u.laplacian)
        Js.append(J), widths.append(u.shape[-1]), flags.append(isinstance(t, LazyBroadcast))
    cat = lambda ts: ts[0] if len(ts) == 1 else torch.cat(ts, dim=-1)
    y, Jy, lapy = K.dense_act_parts(act, cat(xs), cat(ls), Js, widths, flags, group, Wt, bt, param, res, pre)
    out = FwdLaplArray(y, FwdJacobian(Jy, None), lapy)
    if residual is not None and res is None:
        out = _LAPLACE_FN_REGISTRY['add']((residual, out), {}, thr)
    return out


def layer_norm_rule(args, kwargs, sparsity_threshold):
    """Fused rule of ``layer_norm(h, gamma, beta, eps)`` over the last axis -- a custom
    registered function in the way the reference registers its attention kernel
    (folx/experimental/pallas/attention/__init__.py:45).  The fused kernel applies when the
    Jacobian is dense, or sparse with a mask that is constant along the feature axis and
    lists no index twice (every op of the chain then keeps the rows and the mask); other
    inputs go through the chain of primitive rules."""
    h, gamma, beta = args
    eps = float(kwargs.get('eps', 1e-5))
    F = h.shape[-1]
    mask = h.jacobian.x0_idx
    fusable = F % 4 == 0 and F <= 1024
    if fusable and mask is not None:
        first = np.take(mask, [0], axis=-1)
        fusable = bool((mask == first).all()) and not ia.has_duplicates(mask)
    if not fusable:
        from . import numpy as fnp

        mu = fnp.mean(h, axis=-1, keepdims=True)
        c = fnp.subtract(h, mu)
        var = fnp.mean(fnp.square(c), axis=-1, keepdims=True)
        y = fnp.multiply(c, fnp.rsqrt(fnp.add(var, eps)))
        if gamma is not None:
            y = fnp.multiply(y, gamma)
        return y if beta is None else fnp.add(y, beta)
    dev = h.x.device
    g = None if gamma is None else so.device_const(gamma, dev)
    b = None if beta is None else so.device_const(beta, dev)
    y, Jy, lapy = K.layernorm(h.x, h.jacobian.data, h.laplacian, g, b, eps)
    return FwdLaplArray(y, FwdJacobian(Jy, mask), lapy)


def exp_envelope_rule(args, kwargs, sparsity_threshold):
    """Fused rule of ``exp_envelope(d, sigma, pi) = sum_I pi[I, o] exp(-sigma[I, o] d[..., I])``,
    a custom registered function like ``layer_norm``.  The fused kernel applies when the
    Jacobian of ``d`` is dense, or sparse with a mask that is constant along the last axis and
    lists no index twice; other inputs go through the chain of primitive rules
    (broadcast, mul, neg, exp, mul, reduce_sum), which also defines the result."""
    d, sigma, pi = args
    nI, O = (int(v) for v in sigma.shape)
    fusable = _is(d) and K.exp_envelope_supported(nI, O) and d.shape[-1] == nI
    mask = d.jacobian.x0_idx if _is(d) else None
    if fusable and mask is not None:
        first = np.take(mask, [0], axis=-1)
        fusable = bool((mask == first).all()) and not ia.has_duplicates(mask)
    if not fusable:
        from . import numpy as fnp

        e = fnp.exp(fnp.negative(fnp.multiply(fnp.expand_dims(d, -1), sigma)))
        return fnp.sum(fnp.multiply(e, pi), axis=-2)
    dev = d.x.device
    y, Jy, lapy = K.exp_envelope(d.x, d.jacobian.data, d.laplacian, so.device_const(sigma, dev),
                                 so.device_const(pi, dev))
    new_mask = None
    if mask is not None:
        first = np.take(np.broadcast_to(mask, (mask.shape[0], *d.shape)), [0], axis=-1)
        new_mask = np.broadcast_to(first, (mask.shape[0], *d.shape[:-1], O))
    return FwdLaplArray(y, FwdJacobian(Jy, new_mask), lapy)


# --------------------------------------------------------------------------------------
# reductions
# --------------------------------------------------------------------------------------


def _norm_axes(axes, nd):
    if axes is None:
        return tuple(range(nd))
    if isinstance(axes, int):
        axes = (axes,)
    return tuple(sorted(set(a % nd for a in axes)))


def _reduce_tensor(t: torch.Tensor, lead: int, axes, alpha=1.0, window=None) -> torch.Tensor:
    """Sum ``t`` over logical ``axes``; ``lead`` = number of leading non-logical axes.
    ``window = (lo, hi)`` (one axis only) sums that part of the axis."""
    shape = list(t.shape)
    assert window is None or len(axes) == 1
    for ax in sorted(axes, reverse=True):
        full_ax = ax + lead
        outer = int(np.prod(shape[:full_ax], dtype=np.int64))
        red = shape[full_ax]
        inner = int(np.prod(shape[full_ax + 1 :], dtype=np.int64))
        t = K.reduce_sum(t.contiguous().reshape(-1), 1, outer, red, inner, alpha, window)
        alpha = 1.0
        del shape[full_ax]
        t = t.reshape(shape)
    return t


def reduce_sum(args, kwargs, sparsity_threshold):
    """``reduce_sum`` (SUMMATION, folx/wrapped_functions.py:388-392).  Dense: the same sum
    on x, rows and lap.  Sparse (``sparse_sum_jvp``, folx/jvp.py:89-176): static output
    mask, rows gathered into their output slots; past the threshold the rows are summed
    straight into the dense Jacobian (:128-140).

    ``kwargs['window'] = (lo, hi)`` (one axis): the sum of that slice of the axis, read in place
    (a ``slice`` whose only consumer is the sum).  ``kwargs['scale']``: a constant factor applied
    in the same launches (the ``1 / n`` of a mean; LINEAR, folx/wrapped_functions.py:361-376)."""
    (a,) = args
    scale = float(kwargs.get('scale', 1.0))
    if not _is(a):
        if isinstance(a, BatchedArray):
            axes = _norm_axes(kwargs.get('axes'), a.ndim)
            return BatchedArray(_reduce_tensor(a.data, 1, axes, scale))
        return scale * np.sum(np.asarray(a), axis=kwargs.get('axes'))
    axes = _norm_axes(kwargs.get('axes'), a.ndim)
    if len(axes) == 0:
        return a if scale == 1.0 else _affine_const(a, scale, mul=True, alpha=1.0, beta=0.0)
    window = kwargs.get('window')
    if window is not None:
        assert len(axes) == 1
        window = (int(window[0]), int(window[1]))
        assert 0 <= window[0] <= window[1] <= a.shape[axes[0]]
    x = _reduce_tensor(a.x, 1, axes, scale, window)
    lap = _reduce_tensor(a.laplacian, 1, axes, scale, window)
    J, mask = a.jacobian.data, a.jacobian.x0_idx
    if mask is None:
        return FwdLaplArray(x, FwdJacobian(_reduce_tensor(J, 2, axes, scale, window), None), lap)

    k = mask.shape[0]
    mask = np.broadcast_to(mask, (k, *a.shape))
    if window is not None:
        # the index frame of the sum is the one of the slice (folx/jvp.py:108-146 on the sliced mask)
        cut = tuple(slice(*window) if i == axes[0] + 1 else slice(None) for i in range(mask.ndim))
        mask_w = mask[cut]
    else:
        mask_w = mask
    idx_out, slot = ia.sum_out_mask(mask_w, axes)
    if idx_out.shape[0] > sparsity_threshold:
        logging.info(
            f'reduce_sum: output ({idx_out.shape[0]}) reaches sparsity threshold '
            f'({sparsity_threshold}); switching to dense'
        )
        n_out = int(mask.max()) + 1
        slot, out_mask = mask_w, None
    else:
        n_out, out_mask = idx_out.shape[0], idx_out
    red_ax = [ax + 1 for ax in axes]
    first = slot
    for ax in red_ax:
        first = np.take(first, [0], axis=ax)
    kept_shape = [n for i, n in enumerate(a.shape) if i not in axes]
    if (slot == first).all():
        # every row keeps one slot along the reduced axes: reduce rows, then re-slot
        Jr = _reduce_tensor(J, 2, axes, scale, window)
        slot_c = first.reshape(k, *kept_shape)
        ident = n_out == k and (slot_c == np.arange(k).reshape(k, *([1] * (slot_c.ndim - 1)))).all()
        Jo = Jr if ident else so.materialize(Jr, slot_c, n_out)
    elif len(axes) == 1:
        # slots vary along the reduced axis: gather (row, entry of the axis) pairs into their slots, the
        # data read where it lies (no slice of the window, no permuted copy)
        Jo = so.materialize_reduced(J, slot, n_out, axes[0], a.shape, window, scale)
    else:
        # fold the reduced axes into the row axis, then gather (rows, reduced) -> slots
        nd = a.ndim
        kept = [i for i in range(nd) if i not in axes]
        perm = [0] + [ax + 2 for ax in axes] + [1] + [i + 2 for i in kept]
        R = int(np.prod([a.shape[ax] for ax in axes], dtype=np.int64))
        Jp = J.permute(*perm).contiguous().reshape(k * R, a.B, *[a.shape[i] for i in kept])
        sp = np.transpose(slot, [0] + [ax + 1 for ax in axes] + [i + 1 for i in kept])
        sp = sp.reshape(k * R, *[a.shape[i] for i in kept])
        Jo = so.materialize(Jp, sp, n_out)
        if scale != 1.0:
            Jo = _scale_rows(Jo, Jo.shape[0], scale)
    return FwdLaplArray(x, FwdJacobian(Jo, out_mask), lap)


# --------------------------------------------------------------------------------------
# indexing rules: the op is applied to x, rows, lap and to the mask alike
# (sparse_index_jvp, folx/jvp.py:330-413)
# --------------------------------------------------------------------------------------


def _index_rule(fn_t, fn_m):
    """fn_t(tensor, lead) applies the op to a tensor with ``lead`` leading non-logical
    axes; fn_m(mask) applies it to a host mask (one leading row axis)."""

    def apply(a: FwdLaplArray) -> FwdLaplArray:
        mask = a.jacobian.x0_idx
        return FwdLaplArray(
            fn_t(a.x, 1).contiguous(),
            FwdJacobian(fn_t(a.jacobian.data, 2).contiguous(), None if mask is None else fn_m(mask)),
            fn_t(a.laplacian, 1).contiguous(),
        )

    return apply


def _const_index(a, fn_t):
    if isinstance(a, BatchedArray):
        return BatchedArray(fn_t(a.data, 1).contiguous())
    t = torch.as_tensor(np.asarray(a))
    return fn_t(t, 0).numpy()


def reshape_rule(args, kwargs, sparsity_threshold):
    (a,) = args
    shape = tuple(kwargs['new_sizes'])
    fn_t = lambda t, lead: t.reshape(*t.shape[:lead], *shape)
    if not _is(a):
        return _const_index(a, fn_t)
    return _index_rule(fn_t, lambda m: m.reshape(m.shape[0], *shape))(a)


def transpose_rule(args, kwargs, sparsity_threshold):
    (a,) = args
    perm = tuple(kwargs['permutation'])
    fn_t = lambda t, lead: t.permute(*range(lead), *[p + lead for p in perm])
    if not _is(a):
        return _const_index(a, fn_t)
    return _index_rule(fn_t, lambda m: np.transpose(m, (0, *[p + 1 for p in perm])))(a)


def rev_rule(args, kwargs, sparsity_threshold):
    """``lax.rev``: reverse along ``dimensions`` (INDEXING, folx/wrapped_functions.py:505-507)."""
    (a,) = args
    dims = tuple(kwargs['dimensions'])
    fn_t = lambda t, lead: torch.flip(t, [d + lead for d in dims])
    if not _is(a):
        return _const_index(a, fn_t)
    return _index_rule(fn_t, lambda m: np.flip(m, tuple(d + 1 for d in dims)))(a)


def _values_only(torch_fn, np_fn):
    """Piecewise-constant functions (floor, ceil, round, comparisons): the result carries no
    derivatives (``warp_without_fwd_laplacian``, folx/wrapped_functions.py:446-448, :538-551)."""

    def rule(args, kwargs, sparsity_threshold):
        vals, like = [], None
        for a in args:
            t = a.x if _is(a) else (a.data if isinstance(a, BatchedArray) else None)
            like = t if t is not None and like is None else like
            vals.append(t if t is not None else a)
        if like is None:
            return np_fn(*[np.asarray(v) for v in vals])
        tens = [v if isinstance(v, torch.Tensor) else so.device_const(np.asarray(v, dtype=np.float32), like.device)
                for v in vals]
        return BatchedArray(torch_fn(*tens).to(torch.float32))

    return rule


def broadcast_in_dim_rule(args, kwargs, sparsity_threshold):
    """``broadcast_in_dim(shape, broadcast_dimensions)`` as in lax."""
    (a,) = args
    shape = tuple(kwargs['shape'])
    bdims = tuple(kwargs['broadcast_dimensions'])

    def mid_shape(src):
        mid = [1] * len(shape)
        for i, d in enumerate(bdims):
            mid[d] = src[i]
        return mid

    def fn_t(t, lead):
        mid = mid_shape(t.shape[lead:])
        return t.reshape(*t.shape[:lead], *mid).expand(*t.shape[:lead], *shape)

    if not _is(a):
        return _const_index(a, fn_t)
    fn_m = lambda m: np.broadcast_to(m.reshape(m.shape[0], *mid_shape(m.shape[1:])), (m.shape[0], *shape))
    return _index_rule(fn_t, fn_m)(a)


def _canon_index(idx, nd):
    if not isinstance(idx, tuple):
        idx = (idx,)
    if any(i is Ellipsis for i in idx):
        pos = [n for n, i in enumerate(idx) if i is Ellipsis][0]
        n_real = len([i for i in idx if i is not None and i is not Ellipsis])
        idx = idx[:pos] + (slice(None),) * (nd - n_real) + idx[pos + 1 :]
    for i in idx:
        if not (isinstance(i, (int, np.integer, slice)) or i is None):
            raise TypeError('only static basic indexing (ints, slices, None, ...) is supported')
    return idx


def _has_index_arrays(idx) -> bool:
    idx = idx if isinstance(idx, tuple) else (idx,)
    return any(isinstance(i, (np.ndarray, list, torch.Tensor)) for i in idx)


def _take_positions(a, idx):
    """Indexing with static integer arrays (the ``gather`` primitive under
    ``sparse_index_jvp``, folx/jvp.py:330-413): every output element reads one static
    position, so values, Jacobian rows, Laplacian and mask are all re-indexed alike."""
    shape = _logical_shape(a)
    idx = tuple(np.asarray(i.cpu() if isinstance(i, torch.Tensor) else i) if isinstance(i, (list, torch.Tensor))
                else i for i in (idx if isinstance(idx, tuple) else (idx,)))
    pos = ia.index_positions(shape, idx)
    if (pos < 0).any():
        raise IndexError('index out of bounds in a static integer-array index')
    if not _is(a):
        if isinstance(a, BatchedArray):
            flat = a.data.reshape(a.B, -1)
            t = so.device_table(pos.reshape(-1, 1), flat.device)
            return BatchedArray(K.gather_cols(flat.contiguous(), t).reshape(a.B, *pos.shape))
        return np.asarray(a).reshape(-1)[pos]
    B, dev = a.B, a.x.device
    k = a.jacobian.data.shape[0]
    S = int(np.prod(shape, dtype=np.int64))
    t = so.device_table(pos.reshape(-1, 1), dev)
    x = K.gather_cols(a.x.reshape(B, S), t).reshape(B, *pos.shape)
    J = K.gather_cols(a.jacobian.data.reshape(k * B, S), t).reshape(k, B, *pos.shape)
    L = K.gather_cols(a.laplacian.reshape(B, S), t).reshape(B, *pos.shape)
    mask = a.jacobian.x0_idx
    if mask is not None:
        mask = np.broadcast_to(mask, (mask.shape[0], *shape)).reshape(mask.shape[0], S)[:, pos]
    return FwdLaplArray(x, FwdJacobian(J, mask), L)


def getitem_rule(args, kwargs, sparsity_threshold):
    """Static indexing: basic (``slice`` / ``squeeze`` / ``expand_dims`` primitives) on
    views, integer arrays (``gather``) through the position-gather kernel."""
    (a,) = args
    if _has_index_arrays(kwargs['idx']):
        return _take_positions(a, kwargs['idx'])
    idx = _canon_index(kwargs['idx'], len(_logical_shape(a)))
    fn_t = lambda t, lead: t[(*([slice(None)] * lead), *idx)]
    if not _is(a):
        return _const_index(a, fn_t)
    return _index_rule(fn_t, lambda m: m[(slice(None), *idx)])(a)


# --------------------------------------------------------------------------------------
# scatter rules (folx/jvp.py:416-673)
# --------------------------------------------------------------------------------------

_SCATTER_BIG = 3.0e38  # stands in for +-inf at positions no update lands on (min / max)


def _scatter_rows(mode: str, op, upd, tpos: np.ndarray, op_size: int, dev):
    """The scatter arithmetic on row stacks that share one row frame.

    op = (x (B, S_op), J (P, B, S_op), lap (B, S_op)) with J possibly None (constant
    operand), upd likewise over the update elements (J None = constant updates).  Every
    operand position gathers the update elements that land on it through a static table
    (``folx_hip_gather_cols``), so the result does not depend on any write order."""
    ox, oJ, oL = op
    ux, uJ, uL = upd
    B = ox.shape[0]
    withJ = [J for J in (oJ, uJ) if J is not None]
    P = withJ[0].shape[0] if withJ else 0

    def gather(table):
        t = so.device_table(table, dev)
        gx = K.gather_cols(ux.contiguous(), t)
        if uJ is None:
            return gx, None, None
        gJ = K.gather_cols(uJ.reshape(P * B, -1), t).reshape(P, B, op_size)
        return gx, gJ, K.gather_cols(uL.contiguous(), t)

    def plus(a, b):
        if a is None or b is None:
            return a if b is None else b
        return so.add_rowstacks(a.contiguous(), b.contiguous())

    if mode == 'add':
        gx, gJ, gL = gather(ia.scatter_source_table(tpos, op_size, last_only=False))
        return plus(ox, gx), plus(oJ, gJ), plus(oL, gL)

    if mode == 'set':
        table = ia.scatter_source_table(tpos, op_size, last_only=True)
        gx, gJ, gL = gather(table)
        keep = so.device_const((table[:, 0] < 0).astype(np.float32).reshape(1, op_size), dev)
        x = K.rows_affine(ox.contiguous(), 1, (B, op_size), (B, op_size), keep, gx, 1.0, 1.0).reshape(B, op_size)
        if oJ is None:
            return x, gJ, gL
        J = K.rows_affine(oJ.contiguous(), P, (B, op_size), (B, op_size), keep, None, 1.0, 0.0)
        L = K.rows_affine(oL.contiguous(), 1, (B, op_size), (B, op_size), keep, None, 1.0, 0.0).reshape(B, op_size)
        return x, plus(J.reshape(P, B, op_size), gJ), plus(L, gL)

    # min / max: fold the update elements in, one table slot at a time; a position without
    # an element in the slot sees +-BIG there, so the running value wins
    table = ia.scatter_source_table(tpos, op_size, last_only=False)
    op_name = 'min' if mode == 'min' else 'max'
    big = _SCATTER_BIG if mode == 'min' else -_SCATTER_BIG
    zJ = lambda: so.zeros((P, B, op_size), dev)
    cx, cJ, cL = ox.contiguous(), (oJ if oJ is not None else zJ()), (oL if oL is not None else so.zeros((B, op_size), dev))
    for s_ in range(table.shape[1]):
        col = table[:, s_ : s_ + 1]
        gx, gJ, gL = gather(col)
        valid = (col[:, 0] >= 0).astype(np.float32).reshape(1, op_size)
        fill = so.device_const((1.0 - valid) * big, dev)
        gx = K.rows_affine(gx, 1, (B, op_size), (B, op_size), so.device_const(valid, dev), fill, 1.0, 1.0)
        gx = gx.reshape(B, op_size)
        if gJ is None:
            gJ, gL = zJ(), so.zeros((B, op_size), dev)
        cx, cJ, cL = K.binary(op_name, cx, cJ.contiguous(), cL.contiguous(), gx, gJ, gL)
    return cx, cJ, cL


def _scatter_rule(mode: str) -> ForwardLaplacian:
    """``operand.at[idx].set / add / min / max(updates)`` with a static index
    (``sparse_scatter_jvp``, folx/jvp.py:474-673).  args = (operand, updates), kwargs
    ``idx``.  The target position of every update element is computed on the host
    (``index_positions``; out-of-range integer indices drop their update, :434-435).

    Sparse Jacobians: the output mask is the per-position union of the operand's
    dependencies (none where a 'set' overwrites, :549-553) and of the updates landing there
    (:536-567); both arguments are re-indexed to that frame (:640-655) and scattered row by
    row.  Past the threshold the rule densifies before or after the scatter, whichever
    moves fewer elements (:582-598).  Adding constants passes the operand's derivatives
    through (:505-509)."""

    def rule(args, kwargs, sparsity_threshold):
        operand, updates = args
        op_shape = _logical_shape(operand)
        tpos = ia.index_positions(op_shape, kwargs['idx'])
        upd_shape = tuple(tpos.shape)
        op_size = int(np.prod(op_shape, dtype=np.int64))
        upd_size = int(np.prod(upd_shape, dtype=np.int64))
        if not _is(operand) and not _is(updates):
            raise NotImplementedError('scatter of constants into constants needs no derivative rule')
        like = operand if _is(operand) else updates
        B, dev = like.B, like.x.device

        def const_rows(c, shape, size):
            if isinstance(c, BatchedArray):
                t = c.data.to(torch.float32)
                return t.reshape(B, *([1] * (len(shape) - c.ndim)), *c.shape).expand(B, *shape).reshape(B, size)
            t = so.device_const(np.broadcast_to(np.asarray(c, dtype=np.float32), shape), dev)
            return t.reshape(1, size).expand(B, size)

        if _is(updates) and tuple(updates.shape) != upd_shape:
            nd = len(upd_shape)
            updates = _pad_logical(updates, nd)
            updates = broadcast_in_dim_rule((updates,), {'shape': upd_shape, 'broadcast_dimensions': range(nd)}, 0)

        if not _is(updates) and mode == 'add':
            x, _, _ = _scatter_rows('add', (operand.x.reshape(B, op_size), None, None),
                                    (const_rows(updates, upd_shape, upd_size), None, None), tpos, op_size, dev)
            return FwdLaplArray(x.reshape(B, *op_shape), operand.jacobian, operand.laplacian)

        trip = [t for t in (operand, updates) if _is(t)]
        sparse = all(t.jacobian.weak for t in trip)
        out_mask, densify_after = None, False
        if sparse:
            out_mask = ia.scatter_out_mask(
                operand.jacobian.x0_idx if _is(operand) else None,
                updates.jacobian.x0_idx if _is(updates) else None, tpos, op_shape, mode == 'set')
            max_out = out_mask.shape[0]
            if max_out > sparsity_threshold:
                n_dense = max(t.jacobian.max_n for t in trip) + 1
                sparse_cost = (max_out + 1) * (upd_size + op_size) + n_dense * op_size
                if sparse_cost >= n_dense * (upd_size + op_size):
                    sparse = False
                else:
                    densify_after = True

        def rows_of(t, shape, size, frame):
            if not _is(t):
                return const_rows(t, shape, size), None, None
            if frame is None:
                J = t.jacobian.dense_array
            else:
                M = frame.shape[0]
                data = _expand_rows(t.jacobian.data, t.jacobian.data.shape[0], (B, *t.shape), (B, *shape))
                J = so.materialize(data.reshape(-1, B, *shape), ia.get_index_mask(
                    np.broadcast_to(t.jacobian.x0_idx, (t.jacobian.x0_idx.shape[0], *shape)), frame), M)
            return t.x.reshape(B, size), J.reshape(J.shape[0], B, size), t.laplacian.reshape(B, size)

        if sparse:
            flat = out_mask.reshape(out_mask.shape[0], op_size)
            upd_frame = np.where(tpos.reshape(-1) >= 0, flat[:, np.maximum(tpos.reshape(-1), 0)], -2)
            op3 = rows_of(operand, op_shape, op_size, out_mask)
            up3 = rows_of(updates, upd_shape, upd_size, upd_frame.reshape(out_mask.shape[0], *upd_shape))
        else:
            op3 = rows_of(operand, op_shape, op_size, None)
            up3 = rows_of(updates, upd_shape, upd_size, None)
            if op3[1] is not None and up3[1] is not None:
                P = max(op3[1].shape[0], up3[1].shape[0])
                op3 = (op3[0], so.pad_rows(op3[1], P), op3[2])
                up3 = (up3[0], so.pad_rows(up3[1], P), up3[2])
        x, J, L = _scatter_rows(mode, op3, up3, tpos, op_size, dev)
        jac = FwdJacobian(J.reshape(J.shape[0], B, *op_shape), out_mask if sparse else None)
        if densify_after:
            jac = jac.as_dense
        return FwdLaplArray(x.reshape(B, *op_shape), jac, L.reshape(B, *op_shape))

    rule.__name__ = f'scatter_{mode}'
    return rule


def concatenate_rule(args, kwargs, sparsity_threshold):
    """``concatenate`` (INDEXING with every operand static-capable,
    folx/wrapped_functions.py:461-466).  All operands sparse: row counts are padded with
    (mask -1, data 0) (``broadcast_dim``, folx/utils.py:453-481) and constants enter as
    all ``-1`` rows (folx/jvp.py:350-372).  Any dense operand: everything densified
    (folx/jvp.py:340-341)."""
    axis = kwargs.get('dimension', kwargs.get('axis', -1))
    trip = [t for t in args if _is(t)]
    if not trip:
        walker = [t for t in args if isinstance(t, BatchedArray)]
        if not walker:
            return np.concatenate([np.asarray(t) for t in args], axis=axis)
        # derivative-free values that differ from walker to walker (and constants among them)
        Bw, devw, ndw = walker[0].data.shape[0], walker[0].data.device, walker[0].ndim
        parts = [t.data if isinstance(t, BatchedArray) else
                 so.device_const(t, devw).reshape(1, *np.shape(t)).expand(Bw, *np.shape(t)) for t in args]
        return BatchedArray(torch.cat(parts, dim=axis % ndw + 1))
    first = trip[0]
    nd, B, dev = first.ndim, first.B, first.x.device
    axis = axis % nd
    all_sparse = all(t.jacobian.weak for t in trip)
    if all_sparse:
        k = max(t.jacobian.data.shape[0] for t in trip)
    else:
        k = max(t.jacobian.dense_array.shape[0] if not t.jacobian.weak else t.jacobian.max_n + 1 for t in trip)
    xs, Js, Ls, Ms = [], [], [], []
    for t in args:
        if _is(t):
            J = t.jacobian.data if all_sparse else t.jacobian.dense_array
            xs.append(t.x), Ls.append(t.laplacian), Js.append(so.pad_rows(J, k))
            if all_sparse:
                m = t.jacobian.x0_idx
                if m.shape[0] < k:
                    m = np.concatenate([m, np.full((k - m.shape[0], *m.shape[1:]), -1, dtype=m.dtype)], 0)
                Ms.append(m)
        else:
            if isinstance(t, BatchedArray):
                c = t.data
            else:
                c = so.device_const(t, dev)
                c = c.reshape(1, *c.shape).expand(B, *c.shape)
            xs.append(c)
            Ls.append(so.zeros(c.shape, dev))
            Js.append(so.zeros((k, *c.shape), dev))
            if all_sparse:
                Ms.append(np.full((k, *c.shape[1:]), -1, dtype=np.int32))
    x = torch.cat(xs, dim=axis + 1)
    J = torch.cat(Js, dim=axis + 2)
    lap = torch.cat(Ls, dim=axis + 1)
    mask = np.concatenate(Ms, axis=axis + 1) if all_sparse else None
    return FwdLaplArray(x, FwdJacobian(J, mask), lap)


# --------------------------------------------------------------------------------------
# derivative-free outputs
# --------------------------------------------------------------------------------------


def stop_gradient_rule(args, kwargs, sparsity_threshold):
    """``warp_without_fwd_laplacian`` (folx/wrapper.py:141-154): derivatives are dropped."""
    (a,) = args
    return BatchedArray(a.x) if _is(a) else a


def sign_rule(args, kwargs, sparsity_threshold):
    (a,) = args
    data = a.x if _is(a) else (a.data if isinstance(a, BatchedArray) else None)
    if data is None:
        return np.sign(np.asarray(a))
    # sign(x) = d|x|/dx, evaluated by the abs rule on a one-row Jacobian of ones
    ones = torch.empty((1, *data.shape), device=data.device, dtype=torch.float32).fill_(1.0)
    _, d1, _ = K.elementwise('abs', data.contiguous(), ones, data.contiguous())
    return BatchedArray(d1[0])


def reduce_max_values(args, kwargs, sparsity_threshold):
    """max over ``axes`` of the values only, returned derivative-free (the
    ``stop_gradient(max)`` shift of logsumexp / softmax)."""
    (a,) = args
    data = a.x if _is(a) else a.data
    nd = data.dim() - 1
    axes = _norm_axes(kwargs.get('axes'), nd)
    shape = list(data.shape)
    t = data
    for ax in sorted(axes, reverse=True):
        f = ax + 1
        outer = int(np.prod(shape[:f], dtype=np.int64))
        inner = int(np.prod(shape[f + 1 :], dtype=np.int64))
        t = K.reduce_max(t.contiguous().reshape(-1), outer, shape[f], inner)
        del shape[f]
        t = t.reshape(shape)
    return BatchedArray(t)


# --------------------------------------------------------------------------------------
# slogdet (kernel family 4) and attention (kernel family 5)
# --------------------------------------------------------------------------------------


_SPARSE_SLOGDET_MAX_RANK = 64        # limits of folx_hip_sparse_slogdet_fwdlap
_SPARSE_SLOGDET_MAX_FACTOR = 2048


def _sparse_slogdet(A):
    """Rank-one-factor shortcut for a sparse Jacobian (``sparse_slogdet``,
    folx/slogdet.py:249-293): returns ``(sign, FwdLaplArray)`` or None when the planner
    declines (dense Jacobian, mask differing between batch positions, dense contraction
    cheaper) or the tables exceed what the kernel holds in LDS."""
    jac = A.jacobian
    if not jac.weak:
        return None
    k = jac.data.shape[0]
    n = A.shape[-1]
    plan = ia.slogdet_plan(jac.x0_idx, k, A.shape, jac.max_n)
    if plan is None:
        return None
    tables, transposed = plan
    C, rank, width = tables['take'].shape
    if n > 32 or rank > _SPARSE_SLOGDET_MAX_RANK or rank * width > _SPARSE_SLOGDET_MAX_FACTOR:
        return None
    dev = A.x.device
    take, cols, rows = ia.slogdet_kernel_tables(tables, transposed, k, n)
    take, cols, rows = (so.device_table(t, dev) for t in (take, cols, rows))
    sign, ld, ldj, ldl = K.sparse_slogdet(A.x.contiguous(), jac.data.contiguous(), A.laplacian.contiguous(),
                                          take, cols, rows, transposed)
    # a determinant depends on every coordinate its matrix is sparse in: dense output
    # (folx/slogdet.py:238-246)
    out_idx = np.broadcast_to(tables['coords'].reshape(C, *([1] * (ld.dim() - 1))), (C, *ld.shape[1:]))
    dense = FwdJacobian(ldj, out_idx.astype(np.int32)).dense_array
    return BatchedArray(sign), FwdLaplArray(ld, FwdJacobian(dense, None), ldl)


def slogdet_wrapper(args, kwargs, sparsity_threshold):
    """``slogdet_wrapper`` (folx/slogdet.py:347-358): returns ``(sign, FwdLaplArray(logdet))``
    with a dense Jacobian, through the rank-one-factor shortcut when the Jacobian's
    sparsity pays (``sparse_slogdet``, :249-293), else ``dense_slogdet`` (:320-344)."""
    (A,) = args
    if not _is(A):
        raise NotImplementedError('slogdet of a constant: call numpy.linalg.slogdet')
    row_axis = kwargs.get('row_axis')
    factor = kwargs.get('factor')
    if A.shape[-1] > K.SMALL_MATRIX_MAX:
        # beyond the one-matrix-per-wavefront kernels: the same rule composed from an any-size inverse
        # and the batched product kernel (folx/slogdet.py:296-317); canonical layout, dense Jacobian
        if factor is not None:
            A = _LAPLACE_FN_REGISTRY['mul']((A, factor), {}, sparsity_threshold)
        if row_axis is not None and row_axis % A.ndim != A.ndim - 2:
            perm = [a for a in range(A.ndim) if a != row_axis % A.ndim]
            perm.insert(A.ndim - 2, row_axis % A.ndim)
            A = transpose_rule((A,), {'permutation': perm}, sparsity_threshold)
        assert A.shape[-1] == A.shape[-2], 'slogdet needs square matrices'
        sign, ld, ldj, ldl = K.slogdet_any(A.x, A.jacobian.dense_array, A.laplacian)
        return BatchedArray(sign), FwdLaplArray(ld, FwdJacobian(ldj, None), ldl)
    if factor is not None:
        # slogdet(A * factor): with a dense A and a sparse factor of the same shape the product is
        # formed inside the slogdet kernel; any other combination is the mul rule first
        fused = None
        if _is(factor) and not A.jacobian.weak and factor.jacobian.weak and tuple(factor.shape) == tuple(A.shape):
            m = np.broadcast_to(factor.jacobian.x0_idx, (factor.jacobian.x0_idx.shape[0], *A.shape))
            k = m.shape[0]
            if (K.slogdet_scaled_supported(A.shape[-1], k) and factor.jacobian.max_n < A.jacobian.data.shape[0]
                    and not ia.has_duplicates(m)):
                fused = (factor.x.contiguous(), factor.jacobian.data.contiguous(), factor.laplacian.contiguous(),
                         so.device_table(np.ascontiguousarray(m.reshape(k, -1)), A.x.device))
        if fused is None:
            A = _LAPLACE_FN_REGISTRY['mul']((A, factor), {}, sparsity_threshold)
        else:
            ra = None if row_axis is None else row_axis % A.ndim
            assert A.shape[ra if ra is not None else -2] == A.shape[-1], 'slogdet needs square matrices'
            sign, ld, ldj, ldl = K.slogdet(A.x.contiguous(), A.jacobian.data.contiguous(), A.laplacian.contiguous(),
                                           None if ra is None else ra + 1, fused)
            return BatchedArray(sign), FwdLaplArray(ld, FwdJacobian(ldj, None), ldl)
    if row_axis is not None and row_axis % A.ndim != A.ndim - 2:
        # matrix rows on another axis than the one before last
        ra = row_axis % A.ndim
        assert ra < A.ndim - 1 and A.shape[ra] == A.shape[-1], 'slogdet needs square matrices'
        if A.jacobian.weak:
            # the sparse planner works on the canonical layout
            perm = [a for a in range(A.ndim) if a != ra]
            perm.insert(A.ndim - 2, ra)
            return slogdet_wrapper((transpose_rule((A,), {'permutation': perm}, sparsity_threshold),), {},
                                   sparsity_threshold)
        sign, ld, ldj, ldl = K.slogdet(A.x.contiguous(), A.jacobian.data.contiguous(), A.laplacian.contiguous(),
                                       ra + 1)
        return BatchedArray(sign), FwdLaplArray(ld, FwdJacobian(ldj, None), ldl)
    assert A.shape[-1] == A.shape[-2], 'slogdet needs square matrices'
    fast = _sparse_slogdet(A)
    if fast is not None:
        return fast
    J = A.jacobian.dense_array
    sign, ld, ldj, ldl = K.slogdet(A.x, J, A.laplacian)
    return BatchedArray(sign), FwdLaplArray(ld, FwdJacobian(ldj, None), ldl)


def inv_wrapper(args, kwargs, sparsity_threshold):
    """Matrix inverse (``inv_wrapper``, folx/linear_solve.py:114-145); dense output."""
    (A,) = args
    if not _is(A):
        raise NotImplementedError('inverse of a constant: call numpy.linalg.inv')
    assert A.shape[-1] == A.shape[-2], 'inv needs square matrices'
    # one matrix per wavefront up to 32 x 32; beyond, the rule composed from an any-size inverse and the
    # batched product kernels
    rule = K.inv if A.shape[-1] <= K.SMALL_MATRIX_MAX else K.inv_any
    C, CJ, CL = rule(A.x.contiguous(), A.jacobian.dense_array.contiguous(), A.laplacian.contiguous())
    return FwdLaplArray(C, FwdJacobian(CJ, None), CL)


def solve_wrapper(args, kwargs, sparsity_threshold):
    """``y = A^-1 b`` (``solve_wrapper``, folx/linear_solve.py:54-111).  ``b`` of rank 1 is a
    vector, anything else a stack of matrices; batch axes broadcast from the right and an
    operand with fewer batch axes gets them inserted behind the Jacobian axis (``_align``,
    :36-51).  Either operand may be constant; Jacobians are densified and zero-extended to
    a common row count (:93-94)."""
    A, b = args
    like = A if _is(A) else b
    if not _is(like):
        raise NotImplementedError('solve of two constants: call numpy.linalg.solve')
    B, dev = like.B, like.x.device
    n_, m_ = _logical_shape(A)[-1], (1 if len(_logical_shape(b)) == 1 else _logical_shape(b)[-1])
    if n_ > K.SMALL_MATRIX_MAX or m_ > K.SMALL_MATRIX_MAX:
        # beyond the one-system-per-wavefront kernel: y = A^-1 b through the inverse rule (any size) and the
        # product rules; b of rank 1 is a vector, as numpy.matmul has it
        from . import numpy as fnp

        with fnp.sparsity_threshold(sparsity_threshold):
            if _is(A):
                Ainv = inv_wrapper((A,), {}, sparsity_threshold)
            elif isinstance(A, (BatchedArray, torch.Tensor)):
                raise NotImplementedError('solve: a walker-varying constant matrix beyond 32 x 32')
            else:
                Ainv = np.linalg.inv(np.asarray(A, dtype=np.float64)).astype(np.float32)
            return force(fnp.matmul(Ainv, b))

    def parts(v):
        if _is(v):
            return v.x, v.jacobian.dense_array, v.laplacian
        if isinstance(v, BatchedArray):
            return v.data.to(torch.float32), None, None
        if not isinstance(v, torch.Tensor):
            v = np.asarray(v, dtype=np.float32)
        return so.device_const(v, dev)[None], None, None

    Ax, AJ, AL = parts(A)
    bx, bJ, bL = parts(b)
    vector = bx.dim() - 1 == 1
    if vector:
        bx = bx.unsqueeze(-1)
        bJ = None if bJ is None else bJ.unsqueeze(-1)
        bL = None if bL is None else bL.unsqueeze(-1)
    nb = max(Ax.dim() - 3, bx.dim() - 3)

    def lift(t, lead):
        if t is None:
            return None
        missing = nb - (t.dim() - lead - 2)
        return t.reshape(*t.shape[:lead], *([1] * missing), *t.shape[lead:])

    Ax, AL, bx, bL = lift(Ax, 1), lift(AL, 1), lift(bx, 1), lift(bL, 1)
    AJ, bJ = lift(AJ, 2), lift(bJ, 2)
    n, m = bx.shape[-2:]
    assert Ax.shape[-1] == n and Ax.shape[-2] == n, 'solve: shapes of A and b do not match'
    batch = tuple(np.broadcast_shapes(tuple(Ax.shape[1:-2]), tuple(bx.shape[1:-2])))
    if AJ is not None and bJ is not None:
        P = max(AJ.shape[0], bJ.shape[0])
        AJ, bJ = so.pad_rows(AJ, P), so.pad_rows(bJ, P)
    P = (AJ if AJ is not None else bJ).shape[0]
    full_A, full_b = (B, *batch, n, n), (B, *batch, n, m)
    ex = lambda t, shape: None if t is None else t.expand(*shape).contiguous()
    y, yJ, yL = K.solve(ex(Ax, full_A), ex(AJ, (P, *full_A)), ex(AL, full_A),
                        ex(bx, full_b), ex(bJ, (P, *full_b)), ex(bL, full_b), P)
    if vector:
        y, yJ, yL = y.squeeze(-1), yJ.squeeze(-1), yL.squeeze(-1)
    return FwdLaplArray(y, FwdJacobian(yJ, None), yL)


def det_wrapper(args, kwargs, sparsity_threshold):
    """``det`` from the log-determinant (``det_wrapper``, folx/slogdet.py:361-395):
    det = sign exp(logdet), d_c det = det d_c logdet,
    lap det = det (lap logdet + sum_c (d_c logdet)^2) -- which is the ``exp`` rule applied
    to the logdet triplet, scaled by the sign."""
    sign, ld = slogdet_wrapper(args, kwargs, sparsity_threshold)
    e = _LAPLACE_FN_REGISTRY['exp']((ld,), {}, sparsity_threshold)
    return _LAPLACE_FN_REGISTRY['mul']((e, sign), {}, sparsity_threshold)


def _mask_tensor(m, shape, device):
    if m is None:
        return None
    if isinstance(m, BatchedArray):
        m = m.data
    if isinstance(m, torch.Tensor):
        t = m.to(device=device)
        t = (t != 0).to(torch.uint8)
    else:
        t = torch.as_tensor(np.ascontiguousarray(np.asarray(m) != 0).astype(np.uint8)).to(device)
    return t.expand(*shape).contiguous()


def _position_sparse_index(q, k, v):
    """``(index (k, n) int32, P, all_rows_named)`` when q, k, v (per-walker shape (n, H, d)) carry
    the same sparse Jacobian mask, constant over heads and features, in which no input index
    belongs to two sequence positions -- the structure the position-sparse attention kernel
    takes; None otherwise (the Jacobians are then materialised as in the reference)."""
    masks = [t.jacobian.x0_idx for t in (q, k, v)]
    if any(m is None for m in masks) or q.ndim != 3:
        return None
    m0 = np.broadcast_to(masks[0], (masks[0].shape[0], *q.shape))
    for t, m in zip((k, v), masks[1:]):
        if m.shape[0] != m0.shape[0] or tuple(t.shape) != tuple(q.shape):
            return None
        if not np.array_equal(np.broadcast_to(m, m0.shape), m0):
            return None
    index = np.ascontiguousarray(m0[:, :, 0, 0]).astype(np.int32)
    if not (m0 == index[:, :, None, None]).all():
        return None
    n, _, d = q.shape
    if not K.mhsa_sparse_supported(n, d, index.shape[0]):
        return None
    valid = index[index >= 0]
    if valid.size == 0 or np.unique(valid).size != valid.size:
        return None
    P = int(valid.max()) + 1
    return index, P, bool(valid.size == P)


def mhsa_forward_laplacian(args, kwargs, sparsity_threshold):
    """Rule of ``multi_head_self_attention`` (``mhsa_forward_laplacian``,
    folx/experimental/pallas/attention/forward_laplacian.py:27-179).

    args = (q, k, v, mask, input_mask): q, k, v triplets of per-walker shape (n, H, d)
    (the caller scales q by 1/sqrt(d)); ``mask`` (B, n) or (n,) marks real electrons,
    ``input_mask`` (P, B) or (P,) marks active input coordinates; either may be None.
    Jacobians are densified as in the reference (:166-178).
    """
    q, k, v, mask, input_mask = (tuple(args) + (None, None))[:5]
    bias = kwargs.get('bias')
    if not (_is(q) and _is(k) and _is(v)):
        raise NotImplementedError('multi_head_self_attention needs derivative-carrying q, k, v')
    B, dev = q.B, q.x.device
    n = q.shape[0]
    d = q.shape[-1]
    if n > 64 or d > 64 or d % 4 != 0:
        # beyond what the attention kernels are built for: the same function from its primitives
        # (two products of derivative-carrying operands around a softmax), as the reference
        # evaluates attention that is written with einsum (folx/wrapped_functions.py:205-309).
        # Masks (reference_mhsa_kernel, folx/experimental/pallas/attention/mhsa.py:79-94): a score whose
        # query or key is padding is replaced by -1e20 in front of the softmax; Jacobian rows of inactive
        # input coordinates are zero (the kernel never forms them, .../forward_laplacian.py:483-485).
        from . import numpy as fnp

        if input_mask is not None:
            im = input_mask.data if isinstance(input_mask, BatchedArray) else input_mask
            im = im.to(dev) if isinstance(im, torch.Tensor) else torch.as_tensor(np.asarray(im)).to(dev)
            im = (im != 0).to(torch.float32)
            im = im[:, None].expand(im.shape[0], B) if im.dim() == 1 else im

            def drop_rows(t):
                J = t.jacobian.dense_array
                assert im.shape[0] >= J.shape[0], 'input_mask must have one entry per Jacobian row'
                J = so.pad_rows(J, im.shape[0])
                PB, S = J.shape[0] * B, int(np.prod(t.shape, dtype=np.int64))
                Jz = K.rows_affine(J.contiguous().reshape(PB, S), 1, (PB, S), (PB, S), im.reshape(PB, 1).contiguous(), None)
                return FwdLaplArray(t.x, FwdJacobian(Jz.reshape(J.shape), None), t.laplacian)

            q, k, v = drop_rows(q), drop_rows(k), drop_rows(v)
            if bias is not None:
                bias = drop_rows(bias)
        with fnp.sparsity_threshold(sparsity_threshold):
            sc = fnp.einsum('nhd,mhd->hnm', q, k)
            if bias is not None:
                sc = fnp.add(sc, fnp.transpose(bias, (1, 0, 2)))
            if mask is not None:
                m = _mask_tensor(mask, (B, n), dev).to(torch.float32)
                pair = (m[:, None, :, None] * m[:, None, None, :]).expand(B, sc.shape[0], n, n).contiguous()
                sc = fnp.add(fnp.multiply(sc, BatchedArray(pair)), BatchedArray((1.0 - pair) * -1e20))
            return force(fnp.einsum('hnm,mhd->nhd', fnp.softmax(sc, axis=-1), v))
    if bias is None and mask is None and input_mask is None:
        sparse = _position_sparse_index(q, k, v)
        if sparse is not None:
            index, P, all_named = sparse
            o, oj, ol = K.mhsa_sparse(
                q.x, q.jacobian.data, q.laplacian, k.x, k.jacobian.data, k.laplacian, v.x, v.jacobian.data,
                v.laplacian, so.device_table(index, dev), P, all_named)
            return FwdLaplArray(o, FwdJacobian(oj, None), ol)
    trip = (q, k, v) if bias is None else (q, k, v, bias)
    Js = [t.jacobian.dense_array for t in trip]
    P = max(J.shape[0] for J in Js)
    Js = [so.pad_rows(J, P) for J in Js]
    mt = _mask_tensor(mask, (B, n), dev)
    it = None
    if input_mask is not None:
        im = input_mask.data if isinstance(input_mask, BatchedArray) else input_mask
        if not isinstance(im, torch.Tensor):
            im = np.asarray(im)
            if im.ndim == 1:
                im = im[:, None]
        elif im.dim() == 1:
            im = im[:, None]
        assert im.shape[0] == P, 'input_mask must have one entry per Jacobian row'
        it = _mask_tensor(im, (P, B), dev)
    edge = None if bias is None else (bias.x, Js[3], bias.laplacian)
    o, oj, ol = K.mhsa(q.x, Js[0], q.laplacian, k.x, Js[1], k.laplacian, v.x, Js[2], v.laplacian, mt, it, edge)
    return FwdLaplArray(o, FwdJacobian(oj, None), ol)


def mhsea_forward_laplacian(args, kwargs, sparsity_threshold):
    """Rule of ``multi_head_self_edge_attention`` with the reference's argument order
    ``(q, k, e, v, mask, input_mask)`` (``mhsea_forward_laplacian``,
    folx/experimental/pallas/attention/forward_laplacian.py:495-614): scores
    ``q k^T + e`` with an edge-bias triplet ``e`` of per-walker shape (n, H, n)."""
    q, k, e, v, mask, input_mask = (tuple(args) + (None, None))[:6]
    if not _is(e):
        raise NotImplementedError('multi_head_self_edge_attention needs a derivative-carrying edge bias')
    return mhsa_forward_laplacian((q, k, v, mask, input_mask), {**kwargs, 'bias': e}, sparsity_threshold)


# --------------------------------------------------------------------------------------
# registry (names follow folx/wrapped_functions.py:355-561)
# --------------------------------------------------------------------------------------

for _n in ['tanh', 'exp', 'log', 'sqrt', 'rsqrt', 'square', 'logistic', 'sin', 'cos', 'abs', 'log1p',
           'expm1', 'integer_pow', 'silu', 'softplus', 'reciprocal', 'sinh', 'cosh', 'tan', 'asin', 'acos', 'atan',
           'asinh', 'acosh', 'atanh', 'erf', 'erfc', 'erf_inv', 'cbrt', 'pow', 'lgamma', 'digamma']:
    register_function(_n, _unary_rule(_n))
register_function('sigmoid', _unary_rule('logistic'))  # string key, folx/wrapped_functions.py:554
register_function('neg', neg_rule)
register_function('add', _binary_rule('add'))
register_function('add_any', _binary_rule('add'))
register_function('sub', _binary_rule('sub'))
register_function('mul', _binary_rule('mul'))
register_function('div', _binary_rule('div'))
register_function('min', _binary_rule('min'))
register_function('max', _binary_rule('max'))
register_function('dot_general', dot_general)
register_function('layer_norm', layer_norm_rule)
register_function('exp_envelope', exp_envelope_rule)
register_function('reduce_sum', reduce_sum)
register_function('reshape', reshape_rule)
register_function('transpose', transpose_rule)
register_function('rev', rev_rule)
for _n, _tf, _nf in [('floor', torch.floor, np.floor), ('ceil', torch.ceil, np.ceil), ('round', torch.round, np.round),
                     ('gt', torch.gt, np.greater), ('ge', torch.ge, np.greater_equal), ('lt', torch.lt, np.less),
                     ('le', torch.le, np.less_equal), ('eq', torch.eq, np.equal), ('ne', torch.ne, np.not_equal)]:
    register_function(_n, _values_only(_tf, _nf))
for _n, _tf, _nf in [('trunc', torch.trunc, np.trunc), ('is_finite', torch.isfinite, np.isfinite),
                     ('and', lambda a, b: (a != 0) & (b != 0), lambda a, b: np.logical_and(a != 0, b != 0)),
                     ('or', lambda a, b: (a != 0) | (b != 0), lambda a, b: np.logical_or(a != 0, b != 0)),
                     ('xor', lambda a, b: (a != 0) ^ (b != 0), lambda a, b: np.logical_xor(a != 0, b != 0)),
                     ('not', lambda a: a == 0, lambda a: a == 0)]:
    register_function(_n, _values_only(_tf, _nf))  # folx/wrapped_functions.py:546-550
register_function('argmax', lambda args, kw, thr: _values_only(
    lambda a: torch.argmax(a, dim=kw['axis'] + 1 if kw['axis'] >= 0 else kw['axis']),
    lambda a: np.argmax(a, axis=kw['axis']))(args, kw, thr))          # folx/wrapped_functions.py:448-449
register_function('argmin', lambda args, kw, thr: _values_only(
    lambda a: torch.argmin(a, dim=kw['axis'] + 1 if kw['axis'] >= 0 else kw['axis']),
    lambda a: np.argmin(a, axis=kw['axis']))(args, kw, thr))
register_function('broadcast_in_dim', broadcast_in_dim_rule)
register_function('slice', getitem_rule)
register_function('gather', getitem_rule)
register_function('concatenate', concatenate_rule)
register_function('scatter', _scatter_rule('set'))          # primitive names of jax.lax.scatter*_p
register_function('scatter-add', _scatter_rule('add'))
register_function('scatter_min', _scatter_rule('min'))
register_function('scatter_max', _scatter_rule('max'))
register_function('stop_gradient', stop_gradient_rule)
register_function('sign', sign_rule)
register_function('reduce_max_values', reduce_max_values)
register_function('slogdet', slogdet_wrapper)
register_function('det', det_wrapper)
register_function('inv', inv_wrapper)      # string keys, folx/wrapped_functions.py:559-560
register_function('solve', solve_wrapper)
register_function('_multi_head_self_attention', mhsa_forward_laplacian)
register_function('_multi_head_self_edge_attention', mhsea_forward_laplacian)

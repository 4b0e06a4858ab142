"""Thin tensor-level wrappers over the C ABI: torch tensors in, torch tensors out.

torch is used only to own device memory and to name the current HIP stream; every
arithmetic operation happens inside ``libfolx_hip.so``.  All tensors must be float32,
contiguous and on the GPU.  Layout: x (B, *s), jac (P, B, *s), lap (B, *s).
"""

from __future__ import annotations

import ctypes

import numpy as np
import torch

from . import _lib
from ._lib import ACT, BINOP, check


_raw_stream = getattr(torch._C, '_cuda_getCurrentRawStream', None)


def _stream():
    """The current torch stream's handle (the kernels are launched on it).  Asked for on every launch: the
    caller may have switched streams.  The raw getter costs a tenth of ``torch.cuda.current_stream()``,
    which matters for workloads of many short launches."""
    if _raw_stream is not None:
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


class LaunchTimer:
    """Optional per-launch timing with HIP events recorded on the launch stream.

        with LaunchTimer() as lt:
            ...                       # kernels.dense / kernels.mhsa / ... calls
        lt.summary()                  # {(kernel, key): (launches, total_ms)}

    Events bracket each launch on the stream it is issued to, so the elapsed time is the
    kernel's own duration (plus launch gaps of a few microseconds)."""

    active = None

    def __init__(self, only=None):
        self.records = []
        self.only = None if only is None else frozenset(only)  # time these entry points only

    def __enter__(self):
        LaunchTimer.active = self
        return self

    def __exit__(self, *exc):
        LaunchTimer.active = None

    def summary(self):
        torch.cuda.synchronize()
        out = {}
        for name, key, e0, e1 in self.records:
            n, ms = out.get((name, key), (0, 0.0))
            out[(name, key)] = (n + 1, ms + e0.elapsed_time(e1))
        return out


class _timed:
    __slots__ = ('name', 'key', 'e0')

    def __init__(self, name, key):
        self.name, self.key = name, key

    def __enter__(self):
        lt = LaunchTimer.active
        self.e0 = None
        if lt is not None and (lt.only is None or self.name in lt.only):
            self.e0 = torch.cuda.Event(enable_timing=True)
            self.e0.record()

    def __exit__(self, *exc):
        lt = LaunchTimer.active
        if lt is not None and self.e0 is not None:
            e1 = torch.cuda.Event(enable_timing=True)
            e1.record()
            lt.records.append((self.name, self.key, self.e0, e1))


def set_gemm_mode(mode: str):
    """How the wide dense rules form their fp32 products: ``'f32'`` (FP32 matrix instructions, the
    default) or ``'bf16x3'`` (operands split exactly into three bf16 pieces, six exact piece
    products per product accumulated in fp32: same accuracy, the faster matrix pipe).  Process
    wide; the environment variable ``FOLX_AMD_GEMM`` sets it when the library is loaded.  A HIP
    graph captured by ``folx_amd.jit`` keeps the kernels of the mode it was captured under."""
    if mode not in _lib.GEMM_MODE:
        raise ValueError(f'gemm mode {mode!r}: expected one of {sorted(_lib.GEMM_MODE)}')
    _lib.check(_lib.load().folx_hip_set_gemm_mode(_lib.GEMM_MODE[mode]), 'set_gemm_mode')


def get_gemm_mode() -> str:
    code = _lib.load().folx_hip_get_gemm_mode()
    return next(k for k, v in _lib.GEMM_MODE.items() if v == code)


def _p(t):
    if t is None:
        return None
    return ctypes.c_void_p(t.data_ptr())


def _chk(*ts):
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise _lib.FolxHipError('folx_amd kernels need GPU tensors (no CPU fallback)')
        if not t.is_contiguous():
            raise ValueError('non-contiguous tensor passed to a folx_amd kernel')
        if t.dtype not in (torch.float32, torch.int32, torch.uint8):
            raise TypeError(f'unsupported dtype {t.dtype}')


def _dims(*vals):
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def dense(x, jac, lap, W, bias=None, res=None, row_slice=None):
    """x (.., K), jac (P, .., K), lap (.., K), W (K, N) -> triplet with last dim N.
    ``res`` = optional (x, jac, lap) residual triplet of the output shape, added in the
    GEMM epilogue.  ``row_slice = (lo, hi)`` restricts the axis in front of the feature axis
    to [lo, hi): the kernel reads those row groups in place (no copy of the slice)."""
    _chk(x, jac, lap, W, bias)
    rx, rj, rl = res if res is not None else (None, None, None)
    _chk(rx, rj, rl)
    K, N = W.shape
    P = jac.shape[0]
    lead = tuple(x.shape[:-1])
    group = gstride = 0
    xp, jp, lp = _p(x), _p(jac), _p(lap)
    if row_slice is not None:
        lo, hi = row_slice
        n = lead[-1]
        assert 0 <= lo < hi <= n and len(lead) >= 1
        lead = (*lead[:-1], hi - lo)
        group, gstride = hi - lo, n
        off = lo * K * 4  # bytes from the first row of a group of n to row lo
        xp, jp, lp = (ctypes.c_void_p(t.data_ptr() + off) for t in (x, jac, lap))
    R = int(np.prod(lead, dtype=np.int64))
    y = torch.empty((*lead, N), device=x.device, dtype=torch.float32)
    yj = torch.empty((P, *lead, N), device=x.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    with _timed('dense_fwdlap', (R, P, K, N, res is not None)):
        check(
            _lib.load().folx_hip_dense_rows_fwdlap(
                _stream(), xp, jp, lp, _p(W), _p(bias), _p(rx), _p(rj), _p(rl),
                _p(y), _p(yj), _p(yl), R, P, K, N, group, gstride
            ),
            'dense_fwdlap',
        )
    return y, yj, yl


FUSED_ACTS = ('tanh', 'silu', 'logistic', 'sigmoid', 'softplus', 'exp', 'sin', 'cos', 'square')


def _wide_tiles_filled(P, rows, norm):
    """The wide fused kernels cut their tiles into groups of 32 Jacobian rows (16 for the
    activation alone over a multiple of 8 rows, where that wastes less); a last group that is
    mostly empty costs more MFMA work than the fusion saves."""
    if P is None:
        return True
    group = 16 if (not norm and rows % 8 == 0 and -(-P // 16) * 16 < -(-P // 32) * 32) else 32
    return -(-P // group) * group <= 1.125 * P


def dense_act_supported(name, K, N, rows=None, P=None):
    """Shapes and functions the fused dense + activation kernels are built for: narrow layers
    (K, N <= 128), and wide ones (N > 128, K a multiple of 16) over a multiple of 4 rows.
    With ``P`` (Jacobian rows) given, also whether the wide kernel is the faster choice."""
    if name not in FUSED_ACTS:
        return False
    if 4 <= K <= 128 and K % 4 == 0 and 1 <= N <= 128:
        return True
    return (rows is not None and rows > 0 and rows % 4 == 0 and K % 16 == 0 and N > 128 and N % 4 == 0
            and _wide_tiles_filled(P, rows, False))


def dense_act_residual_supported(K, N):
    """Layers whose fused kernel adds a skip connection in its epilogue (the narrow ones)."""
    return 4 <= K <= 128 and K % 4 == 0 and N <= 128


def dense_act(name, x, jac, lap, W, bias=None, param=0.0, res=None):
    """``f(x @ W + bias)`` as one rule: x (.., K), jac (P, .., K), lap (.., K), W (K, N) ->
    the activated triplet with last dim N; the pre-activation triplet is never written.
    ``res`` = (x, jac, lap) of the output's shape is added to the activated result (narrow
    layers only)."""
    _chk(x, jac, lap, W, bias, *(res or ()))
    K, N = W.shape
    P = jac.shape[0]
    lead = tuple(x.shape[:-1])
    R = int(np.prod(lead, dtype=np.int64))
    lib = _lib.load()
    nbytes = int(lib.folx_hip_dense_act_workspace_bytes(R, P, K, N))
    if nbytes < 0:
        check(nbytes, 'dense_act_workspace_bytes')
    ws = torch.empty(nbytes // 4, device=x.device, dtype=torch.float32) if nbytes > 0 else None
    y = torch.empty((*lead, N), device=x.device, dtype=torch.float32)
    yj = torch.empty((P, *lead, N), device=x.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    rx, rj, rl = (None, None, None) if res is None else res
    if res is not None:
        assert tuple(rx.shape) == tuple(y.shape) and tuple(rj.shape) == tuple(yj.shape) and tuple(rl.shape) == tuple(y.shape)
    with _timed('dense_act_fwdlap', (name, R, P, K, N)):
        check(
            lib.folx_hip_dense_act_fwdlap(
                _stream(), ACT[name], float(param), _p(x), _p(jac), _p(lap), _p(W), _p(bias),
                _p(rx), _p(rj), _p(rl), _p(y), _p(yj), _p(yl), R, P, K, N, _p(ws), nbytes
            ),
            f'dense_act_fwdlap[{name}]',
        )
    return y, yj, yl


def dense_act_parts(name, x, lap, jac_parts, widths, broadcast, group, W, bias=None, param=0.0, res=None, pre=None):
    """``dense_act`` of a wide layer whose Jacobian operand is the concatenation along the
    feature axis of ``jac_parts`` (never formed): part i is (P, rows_i, widths[i]) with rows_i
    the layer's rows, or one row per ``group`` of them where ``broadcast[i]``; x and lap are
    the concatenated arrays (.., K); ``res`` = (x, jac, lap) of the output's shape is added to
    the activated result; ``pre`` = (x (rows / group, N), jac (P, rows / group, N), lap) is added
    to the pre-activation triplet, one row per ``group`` of the layer's rows."""
    _chk(x, lap, W, bias, *jac_parts, *(res or ()), *(pre or ()))
    K, N = W.shape
    assert sum(widths) == K and x.shape[-1] == K
    P = jac_parts[0].shape[0]
    lead = tuple(x.shape[:-1])
    R = int(np.prod(lead, dtype=np.int64))
    n = len(jac_parts)
    for J, w, bc in zip(jac_parts, widths, broadcast):
        assert J.is_contiguous() and J.shape[0] == P and J.numel() == P * (R // group if bc else R) * w
    x, lap = x.contiguous(), lap.contiguous()
    lib = _lib.load()
    nbytes = int(lib.folx_hip_dense_act_workspace_bytes(R, P, K, N))
    if nbytes < 0:
        check(nbytes, 'dense_act_workspace_bytes')
    ws = torch.empty(max(nbytes // 4, 1), device=x.device, dtype=torch.float32)
    y = torch.empty((*lead, N), device=x.device, dtype=torch.float32)
    yj = torch.empty((P, *lead, N), device=x.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    rx, rj, rl = (None, None, None) if res is None else res
    if res is not None:
        assert rx.is_contiguous() and rj.is_contiguous() and rl.is_contiguous()
        assert tuple(rx.shape) == tuple(y.shape) and tuple(rj.shape) == tuple(yj.shape)
    px, pj, pl = (None, None, None) if pre is None else pre
    if pre is not None:
        assert px.is_contiguous() and pj.is_contiguous() and pl.is_contiguous() and R % group == 0
        assert px.numel() == (R // group) * N and pj.numel() == P * (R // group) * N and pl.numel() == px.numel()
    ptrs = (ctypes.c_void_p * n)(*[J.data_ptr() for J in jac_parts])
    wd = (ctypes.c_int32 * n)(*[int(w) for w in widths])
    bc = (ctypes.c_int32 * n)(*[int(bool(b)) for b in broadcast])
    with _timed('dense_act_fwdlap', (name, R, P, K, N)):
        check(
            lib.folx_hip_dense_act_parts_fwdlap(
                _stream(), ACT[name], float(param), _p(x), _p(lap), n, ptrs, wd, bc, int(group), _p(W), _p(bias),
                _p(rx), _p(rj), _p(rl), _p(px), _p(pj), _p(pl), _p(y), _p(yj), _p(yl), R, P, N, _p(ws), nbytes
            ),
            f'dense_act_parts_fwdlap[{name}]',
        )
    return y, yj, yl


def norm_dense_supported(name, K, N, rows, P=None):
    """Shapes and functions ``norm_dense`` is built for (``name`` None: no activation); with
    ``P`` (Jacobian rows) given, also whether it is the faster choice."""
    return ((name is None or name in FUSED_ACTS) and rows > 0 and rows % 4 == 0 and K % 16 == 0 and K <= 512
            and N > 128 and N % 4 == 0 and _wide_tiles_filled(P, rows, True))


def norm_dense(name, x, jac, lap, gamma, beta, eps, W, bias=None, param=0.0):
    """``f(layer_norm(x) @ W + bias)`` as one rule (``name`` None: no ``f``): x (.., K), jac
    (P, .., K), lap (.., K), gamma / beta (K) or None, W (K, N) -> triplet with last dim N."""
    _chk(x, jac, lap, gamma, beta, W, bias)
    K, N = W.shape
    P = jac.shape[0]
    lead = tuple(x.shape[:-1])
    R = int(np.prod(lead, dtype=np.int64))
    act = -1 if name is None else ACT[name]
    lib = _lib.load()
    nbytes = int(lib.folx_hip_norm_dense_workspace_bytes(R, P, K, N, act))
    if nbytes < 0:
        check(nbytes, 'norm_dense_workspace_bytes')
    ws = torch.empty(nbytes // 4, device=x.device, dtype=torch.float32)
    y = torch.empty((*lead, N), device=x.device, dtype=torch.float32)
    yj = torch.empty((P, *lead, N), device=x.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    with _timed('norm_dense_fwdlap', (name, R, P, K, N)):
        check(
            lib.folx_hip_norm_dense_fwdlap(
                _stream(), act, float(param), _p(x), _p(jac), _p(lap), _p(gamma), _p(beta), float(eps), _p(W),
                _p(bias), _p(y), _p(yj), _p(yl), R, P, K, N, _p(ws), nbytes
            ),
            f'norm_dense_fwdlap[{name}]',
        )
    return y, yj, yl


DOT_TWO_KMAX = 128


def dot_two(a, aj, al, b, bj, bl):
    """Batched product of two triplets: a (NB0, NB1, I, Kc), b (NB0, NB1, Kc, J), Jacobians with a
    leading row axis (P, ...), all float32 on the GPU.  The operands may be VIEWS (transposed,
    sliced, head-interleaved): the kernel addresses them through their strides; only the
    Jacobians must share the strides of their values.  Returns contiguous y (NB0, NB1, I, J),
    y_jac (P, NB0, NB1, I, J), y_lap."""
    for t in (a, aj, al, b, bj, bl):
        assert t.is_cuda and t.dtype == torch.float32
    NB0, NB1, I, Kc = a.shape
    J = b.shape[-1]
    P = aj.shape[0]
    assert tuple(b.shape) == (NB0, NB1, Kc, J) and tuple(aj.shape) == (P, *a.shape) and tuple(bj.shape) == (P, *b.shape)
    assert al.shape == a.shape and bl.shape == b.shape and Kc <= DOT_TWO_KMAX

    def same_layout(t, u_strides):  # u is addressed with t's strides
        return all(st == su for st, su, n in zip(t.stride(), u_strides, t.shape) if n > 1)

    assert (same_layout(a, al.stride()) and same_layout(b, bl.stride())
            and (P == 0 or (same_layout(a, aj.stride()[1:]) and same_layout(b, bj.stride()[1:])))), \
        'dot_two: value, Laplacian and Jacobian rows of an operand must share one layout'
    y = torch.empty((NB0, NB1, I, J), device=a.device, dtype=torch.float32)
    yj = torch.empty((P, NB0, NB1, I, J), device=a.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    strides = (ctypes.c_int64 * 10)(*a.stride(), aj.stride(0) if P else 0, b.stride(0), b.stride(1), b.stride(2),
                                    b.stride(3), bj.stride(0) if P else 0)
    with _timed('dot_two_fwdlap', (NB0 * NB1, I, J, Kc, P)):
        check(
            _lib.load().folx_hip_dot_two_fwdlap(
                _stream(), _p(a), _p(aj), _p(al), _p(b), _p(bj), _p(bl), _p(y), _p(yj), _p(yl),
                NB0, NB1, I, J, Kc, P, strides,
            ),
            'dot_two_fwdlap',
        )
    return y, yj, yl


def dot_const(a, aj, al, W):
    """Batched product of a triplet with an operand that carries no derivatives: a (B, Bt, I, Kc), aj (P, B, Bt, I, Kc),
    al like a; W (Bt, Kc, J) -- a constant with a batch axis, read once per batch element (walker stride 0) -- or
    W (B, Bt, Kc, J), one matrix per walker and batch element.  float32 on the GPU; all operands may be views.
    Returns contiguous y (B, Bt, I, J), y_jac (P, B, Bt, I, J), y_lap.  Contracted lengths beyond the kernel's tile
    depth are cut into slices of the contracted axis (views) whose products are added."""
    for t in (a, aj, al, W):
        assert t.is_cuda and t.dtype == torch.float32
    B, Bt, I, Kc = a.shape
    J = W.shape[-1]
    P = aj.shape[0]
    if W.dim() == 3:
        W = W.unsqueeze(0).expand(B, *W.shape)   # stride 0 along the walkers
    assert tuple(W.shape) == (B, Bt, Kc, J) and tuple(aj.shape) == (P, *a.shape) and al.shape == a.shape

    def same_layout(t, u_strides):
        return all(st == su for st, su, n in zip(t.stride(), u_strides, t.shape) if n > 1)

    if not (same_layout(a, al.stride()) and (P == 0 or same_layout(a, aj.stride()[1:]))):
        a, aj, al = a.contiguous(), aj.contiguous(), al.contiguous()
    out = None
    for k0 in range(0, max(Kc, 1), DOT_TWO_KMAX):
        k1 = min(Kc, k0 + DOT_TWO_KMAX)
        ac, ajc, alc, Wc = a[..., k0:k1], aj[..., k0:k1], al[..., k0:k1], W[:, :, k0:k1, :]
        y = torch.empty((B, Bt, I, J), device=a.device, dtype=torch.float32)
        yj = torch.empty((P, B, Bt, I, J), device=a.device, dtype=torch.float32)
        yl = torch.empty_like(y)
        strides = (ctypes.c_int64 * 10)(*ac.stride(), ajc.stride(0) if P else 0, *Wc.stride(), 0)
        with _timed('dot_const_fwdlap', (B * Bt, I, J, k1 - k0, P)):
            check(
                _lib.load().folx_hip_dot_two_fwdlap(
                    _stream(), _p(ac), _p(ajc), _p(alc), _p(Wc), None, None, _p(y), _p(yj), _p(yl),
                    B, Bt, I, J, k1 - k0, P, strides,
                ),
                'dot_two_fwdlap (constant operand)',
            )
        out = (y, yj, yl) if out is None else tuple(_add_flat(o, n) for o, n in zip(out, (y, yj, yl)))
    return out


def _add_flat(a, b, alpha=1.0, beta=1.0):
    """alpha a + beta b for two equally shaped contiguous tensors (one flat affine launch)."""
    n = a.numel()
    if n == 0:
        return a
    return rows_affine(a.reshape(n), 1, (n,), (n,), None, b.reshape(n), alpha, beta).reshape(a.shape)


def inv_values(A):
    """A (NM, n, n) contiguous -> A^-1 (NM, n, n), sign (NM,), log|det| (NM,): Gauss-Jordan with partial pivoting,
    any n."""
    _chk(A)
    NM, n, _ = A.shape
    Ainv = torch.empty_like(A)
    sign = torch.empty(NM, device=A.device, dtype=torch.float32)
    ld = torch.empty_like(sign)
    with _timed('inv_values', (NM, n)):
        check(_lib.load().folx_hip_inv_values(_stream(), _p(A), _p(Ainv), _p(sign), _p(ld), NM, n), 'inv_values')
    return Ainv, sign, ld


def trace_pair(M):
    """M (R, n, n) contiguous -> tr M (R,), tr(M M) (R,)."""
    _chk(M)
    R, n, _ = M.shape
    tr = torch.empty(R, device=M.device, dtype=torch.float32)
    trsq = torch.empty_like(tr)
    with _timed('trace_pair', (R, n)):
        check(_lib.load().folx_hip_trace_pair(_stream(), _p(M), _p(tr), _p(trsq), R, n), 'trace_pair')
    return tr, trsq


def _inverse_times_rows(A, AJ, AL):
    """A^-1 and, TRANSPOSED, M_c = A^-1 dA_c and L = A^-1 lap_A for matrices of any size: the batched product
    (dA_c)^T A^-T with the derivative-carrying operand on the left, both read as transposed views.
    A (NM, n, n), AJ (P, NM, n, n), AL (NM, n, n) contiguous -> Ainv, sign, logdet, Mt (P, NM, n, n), Lt (NM, n, n)."""
    Ainv, sign, ld = inv_values(A)
    t = lambda v: v.unsqueeze(-3).transpose(-1, -2)     # (.., NM, 1, n, n), matrices transposed
    _, Mt, Lt = dot_const(t(A), t(AJ), t(AL), t(Ainv))
    return Ainv, sign, ld, Mt.squeeze(-3), Lt.squeeze(-3)


def slogdet_any(A, AJ, AL):
    """The slogdet rule for matrices of any size, composed (folx/slogdet.py:296-317): A (.., n, n), AJ (P, .., n, n),
    AL like A -> sign (..), logdet (..), jac (P, ..), lap (..).  jac_c = tr M_c and
    lap = tr(A^-1 lap_A) - sum_c tr(M_c M_c) with M_c = A^-1 dA_c from the batched product kernel."""
    _chk(A, AJ, AL)
    n, P, lead = A.shape[-1], AJ.shape[0], tuple(A.shape[:-2])
    NM = int(np.prod(lead, dtype=np.int64))
    _, sign, ld, Mt, Lt = _inverse_times_rows(A.contiguous().reshape(NM, n, n), AJ.contiguous().reshape(P, NM, n, n),
                                              AL.contiguous().reshape(NM, n, n))
    trl, _ = trace_pair(Lt)
    if P > 0:
        trj, sqj = trace_pair(Mt.reshape(P * NM, n, n))
        lap = _add_flat(trl, reduce_sum(sqj, 1, 1, P, NM).reshape(NM), 1.0, -1.0)
    else:
        trj, lap = torch.empty(0, device=A.device, dtype=torch.float32), trl
    return sign.reshape(lead), ld.reshape(lead), trj.reshape(P, *lead), lap.reshape(lead)


def inv_any(A, AJ, AL):
    """The inverse rule for matrices of any size, composed (folx/linear_solve.py:114-145): C = A^-1,
    C_jac[c] = -M_c C, C_lap = (2 sum_c M_c M_c - C lap_A) C with M_c = C dA_c.  Same shapes as ``inv``."""
    _chk(A, AJ, AL)
    n, P, lead = A.shape[-1], AJ.shape[0], tuple(A.shape[:-2])
    NM = int(np.prod(lead, dtype=np.int64))
    C, _, _, Mt, Lt = _inverse_times_rows(A.contiguous().reshape(NM, n, n), AJ.contiguous().reshape(P, NM, n, n),
                                          AL.contiguous().reshape(NM, n, n))
    four = lambda v: v.unsqueeze(-3)                     # (.., NM, 1, n, n)
    if P > 0:
        # 2 sum_c (M_c M_c)^T = 2 sum_c Mt_c Mt_c: the second-order term of the two-operand product rule
        zero = torch.zeros_like(Lt)
        S2t = None
        for k0 in range(0, n, DOT_TWO_KMAX):   # contracted axis in slices the product kernel takes
            k1 = min(n, k0 + DOT_TWO_KMAX)
            _, _, part = dot_two(four(zero)[..., k0:k1], four(Mt)[..., k0:k1], four(zero)[..., k0:k1],
                                 four(zero)[..., k0:k1, :], four(Mt)[..., k0:k1, :], four(zero)[..., k0:k1, :])
            S2t = part if S2t is None else _add_flat(S2t, part)
        Zt = _add_flat(Lt, S2t.reshape(Lt.shape), 1.0, -1.0)   # (L - 2 sum_c M_c M_c)^T
    else:
        Zt = Lt
    negC = _add_flat(C, C, -1.0, 0.0)
    t = lambda v: four(v).transpose(-1, -2)
    _, CJ, CL = dot_const(t(Zt), t(Mt), t(Zt), four(negC))   # M_c (-C),  (L - 2 sum M M) (-C)
    return C.reshape(A.shape), CJ.reshape(AJ.shape), CL.reshape(AL.shape)


def elementwise(name, x, jac, lap, param=0.0, inplace=False):
    _chk(x, jac, lap)
    P = jac.shape[0]
    S = x.numel()
    if inplace:
        y, yj, yl = x, jac, lap
    else:
        y, yj, yl = torch.empty_like(x), torch.empty_like(jac), torch.empty_like(lap)
    with _timed('elementwise_fwdlap', (name, S, P)):
        check(
            _lib.load().folx_hip_elementwise_fwdlap(
                _stream(), ACT[name], float(param), _p(x), _p(jac), _p(lap), _p(y), _p(yj), _p(yl), S, P
            ),
            f'elementwise_fwdlap[{name}]',
        )
    return y, yj, yl


def exp_envelope_supported(n_cols, O):
    return 1 <= n_cols <= 8 and O % 4 == 0


def exp_envelope(d, dj, dl, sigma, pi):
    """``sum_I pi[I, o] exp(-sigma[I, o] d[..., I])``: d (.., nI), dj (P, .., nI), sigma / pi
    (nI, O) -> triplet with last dim O."""
    _chk(d, dj, dl, sigma, pi)
    nI, O = sigma.shape
    assert d.shape[-1] == nI and tuple(pi.shape) == (nI, O)
    P = dj.shape[0]
    lead = tuple(d.shape[:-1])
    R = int(np.prod(lead, dtype=np.int64))
    y = torch.empty((*lead, O), device=d.device, dtype=torch.float32)
    yj = torch.empty((P, *lead, O), device=d.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    with _timed('exp_envelope_fwdlap', (R, nI, O, P)):
        check(
            _lib.load().folx_hip_exp_envelope_fwdlap(
                _stream(), _p(d), _p(dj), _p(dl), _p(sigma), _p(pi), _p(y), _p(yj), _p(yl), R, nI, O, P
            ),
            'exp_envelope_fwdlap',
        )
    return y, yj, yl


def layernorm(x, jac, lap, gamma, beta, eps):
    """Fused LayerNorm rule over the last axis."""
    _chk(x, jac, lap, gamma, beta)
    F = x.shape[-1]
    R = x.numel() // F
    P = jac.shape[0]
    y, yj, yl = torch.empty_like(x), torch.empty_like(jac), torch.empty_like(lap)
    with _timed('layernorm_fwdlap', (R, F, P)):
        check(
            _lib.load().folx_hip_layernorm_fwdlap(
                _stream(), _p(x), _p(jac), _p(lap), _p(gamma), _p(beta), _p(y), _p(yj), _p(yl), R, F, P, float(eps)
            ),
            'layernorm_fwdlap',
        )
    return y, yj, yl


def collapse3(out_shape, *strides_list):
    """Collapse a broadcast index space to <= 3 dims.  ``strides_list``: per operand, the
    element strides over ``out_shape`` (0 where broadcast).  Returns (n, [s, ...]) with
    len(n) == 3, or None if more than 3 dims remain."""
    dims = [(int(n), tuple(int(s[i]) for s in strides_list)) for i, n in enumerate(out_shape) if n != 1]
    merged = []
    for n, st in dims:
        if merged:
            pn, pst = merged[-1]
            if all(ps == s * n for ps, s in zip(pst, st)):
                merged[-1] = (pn * n, st)
                continue
        merged.append((n, st))
    if len(merged) > 3:
        return None
    while len(merged) < 3:
        merged.insert(0, (1, tuple(0 for _ in strides_list)))
    n = [m[0] for m in merged]
    per_op = [[m[1][k] for m in merged] for k in range(len(strides_list))]
    return n, per_op


def bstrides(shape, out_shape):
    """Element strides of a contiguous array of ``shape`` broadcast to ``out_shape``."""
    shape = (1,) * (len(out_shape) - len(shape)) + tuple(shape)
    st, acc = [], 1
    for n in reversed(shape):
        st.append(acc)
        acc *= n
    st = st[::-1]
    return [0 if n == 1 and o != 1 else s for n, s, o in zip(shape, st, out_shape)]


def binary(op, a, aj, al, b, bj, bl):
    """Same-frame binary rule with numpy-style broadcasting of the (B, *s) shapes."""
    _chk(a, aj, al, b, bj, bl)
    P = aj.shape[0]
    assert bj.shape[0] == P
    out_shape = torch.broadcast_shapes(a.shape, b.shape)
    # the kernel addresses an operand's Jacobian rows with the strides of its values: rows that were
    # re-indexed at the full output shape take their (smaller) value and Laplacian arrays along
    if tuple(aj.shape[1:]) != tuple(a.shape):
        assert tuple(aj.shape[1:]) == tuple(out_shape), (aj.shape, a.shape, out_shape)
        a, al = a.expand(out_shape).contiguous(), al.expand(out_shape).contiguous()
    if tuple(bj.shape[1:]) != tuple(b.shape):
        assert tuple(bj.shape[1:]) == tuple(out_shape), (bj.shape, b.shape, out_shape)
        b, bl = b.expand(out_shape).contiguous(), bl.expand(out_shape).contiguous()
    col = collapse3(out_shape, bstrides(a.shape, out_shape), bstrides(b.shape, out_shape))
    if col is None:
        a, aj, al = (t.expand(*t.shape[: t.dim() - a.dim()], *out_shape).contiguous() for t in (a, aj, al))
        b, bj, bl = (t.expand(*t.shape[: t.dim() - b.dim()], *out_shape).contiguous() for t in (b, bj, bl))
        col = collapse3(out_shape, bstrides(a.shape, out_shape), bstrides(b.shape, out_shape))
    n, (sa, sb) = col
    y = torch.empty(out_shape, device=a.device, dtype=torch.float32)
    yj = torch.empty((P, *out_shape), device=a.device, dtype=torch.float32)
    yl = torch.empty_like(y)
    with _timed('binary_fwdlap', (op, int(y.numel()), P)):
        check(
            _lib.load().folx_hip_binary_fwdlap(
                _stream(), BINOP[op], _p(a), _p(aj), _p(al), _p(b), _p(bj), _p(bl), _p(y), _p(yj), _p(yl),
                _dims(*n, *sa, *sb), a.numel(), b.numel(), P,
            ),
            f'binary_fwdlap[{op}]',
        )
    return y, yj, yl


def mul_sparse(a, aj, al, b, bj, bl, index):
    """``a * b`` for triplets of one shape (B, *s): ``aj`` dense (P, B, *s), ``bj`` sparse
    (k, B, *s) with ``index`` int32 (k, prod(s)) on the device naming the dense row of each
    slot.  Returns the triplet with P dense rows."""
    _chk(a, aj, al, b, bj, bl, index)
    assert tuple(a.shape) == tuple(b.shape)
    P, k = aj.shape[0], bj.shape[0]
    S = a.numel()
    S_w = S // a.shape[0]
    assert tuple(index.shape) == (k, S_w) and index.dtype == torch.int32
    y, yj, yl = torch.empty_like(a), torch.empty_like(aj), torch.empty_like(a)
    with _timed('mul_sparse_fwdlap', (S, P, k)):
        check(
            _lib.load().folx_hip_mul_sparse_fwdlap(
                _stream(), _p(a), _p(aj), _p(al), _p(b), _p(bj), _p(bl), _p(index), _p(y), _p(yj), _p(yl),
                S, S_w, P, k,
            ),
            'mul_sparse_fwdlap',
        )
    return y, yj, yl


def rows_affine(inp, rows, row_shape, out_shape, c=None, d=None, alpha=1.0, beta=1.0):
    """out[r] = alpha * in[r] * c + beta * d with broadcasting to ``out_shape``.
    ``inp`` holds ``rows`` rows of shape ``row_shape``; c / d are arrays broadcastable to
    ``out_shape``.  Returns a tensor (rows, *out_shape)."""
    _chk(inp, c, d)
    sin = bstrides(row_shape, out_shape)
    sc = bstrides(c.shape, out_shape) if c is not None else [0] * len(out_shape)
    sd = bstrides(d.shape, out_shape) if d is not None else [0] * len(out_shape)
    col = collapse3(out_shape, sin, sc, sd)
    if col is None:
        # a coefficient array that is broadcast along inner axes (e.g. a per-matrix identity against
        # (walker, row, determinant, column)): spell its broadcast out over all axes but the first,
        # then over all axes, until the index space collapses to three dimensions
        for lead in (1, 0):
            def spelled(t):
                if t is None:
                    return None
                full = (1,) * (len(out_shape) - t.dim()) + tuple(t.shape)
                tgt = tuple(full[:lead]) + tuple(out_shape[lead:])
                return t.reshape(full).expand(tgt).contiguous()
            c2, d2 = spelled(c), spelled(d)
            sc = bstrides(c2.shape, out_shape) if c2 is not None else [0] * len(out_shape)
            sd = bstrides(d2.shape, out_shape) if d2 is not None else [0] * len(out_shape)
            col = collapse3(out_shape, sin, sc, sd)
            if col is not None:
                c, d = c2, d2
                break
    if col is None:
        # the INPUT is broadcast along several separate groups of axes: spell the first group out in a pass of its own
        # (a plain broadcast copy, three index dimensions), then come back with one group fewer
        rs = (1,) * (len(out_shape) - len(row_shape)) + tuple(int(v) for v in row_shape)
        grown = [i for i, (a_, o_) in enumerate(zip(rs, out_shape)) if a_ == 1 and o_ != 1]
        if grown:
            first = [grown[0]]
            while first[-1] + 1 in grown:
                first.append(first[-1] + 1)
            mid = tuple(out_shape[i] if i in first else rs[i] for i in range(len(rs)))
            if mid != rs and len(first) < len(grown):
                step = rows_affine(inp, rows, rs, mid)
                return rows_affine(step, rows, mid, out_shape, c, d, alpha, beta)
        raise NotImplementedError(
            f'rows_affine: the input of shape {tuple(row_shape)} broadcast to {tuple(out_shape)} needs more than '
            'three index dimensions; broadcast it with broadcast_to first')
    n, (s_in, s_c, s_d) = col
    out = torch.empty((rows, *out_shape), device=inp.device, dtype=torch.float32)
    in_S = int(np.prod(row_shape, dtype=np.int64))
    with _timed('rows_affine', (rows, int(np.prod(out_shape, dtype=np.int64)))):
        check(
            _lib.load().folx_hip_rows_affine(
                _stream(), _p(inp), _p(out), rows, in_S, _p(c), _p(d), float(alpha), float(beta),
                _dims(*n, *s_in, *s_c, *s_d),
            ),
            'rows_affine',
        )
    return out


def reduce_sum(inp, rows, outer, red, inner, alpha=1.0, window=None):
    """inp (rows, outer, red, inner) -> (rows, outer, inner); ``window = (lo, hi)`` sums that
    part of the reduced axis only."""
    _chk(inp)
    out = torch.empty((rows, outer, inner), device=inp.device, dtype=torch.float32)
    with _timed('reduce_sum', (rows, outer, red, inner)):
        if window is None:
            rc = _lib.load().folx_hip_reduce_sum(_stream(), _p(inp), _p(out), rows, outer, red, inner, float(alpha))
        else:
            lo, hi = window
            rc = _lib.load().folx_hip_reduce_sum_window(_stream(), _p(inp), _p(out), rows, outer, red, int(lo), int(hi),
                                                        inner, float(alpha))
        check(rc, 'reduce_sum')
    return out


def reduce_max(inp, outer, red, inner):
    _chk(inp)
    out = torch.empty((outer, inner), device=inp.device, dtype=torch.float32)
    check(_lib.load().folx_hip_reduce_max(_stream(), _p(inp), _p(out), outer, red, inner), 'reduce_max')
    return out


def gather_rows(data, take, k_out, n_slots, B, S_outer, S_inner):
    """data (k_in, B, S_outer * S_inner); take int32 (k_out, n_slots, S_outer) on device."""
    _chk(data, take)
    k_in = data.shape[0]
    out = torch.empty((k_out, B, S_outer * S_inner), device=data.device, dtype=torch.float32)
    with _timed('gather_rows', (k_in, k_out, n_slots, B, S_outer, S_inner)):
        check(
            _lib.load().folx_hip_gather_rows(
                _stream(), _p(data), _p(take), _p(out), k_in, k_out, n_slots, B, S_outer, S_inner
            ),
            'gather_rows',
        )
    return out


def gather_reduce_rows(data, take, k_out, n_slots, B, O, RED, IV, IC, alpha=1.0):
    """data (k_in, B, O, RED, IV, IC) in its own layout, take int32 (k_out, n_slots, O * IV) with
    entries r * RED + j (or -1) -> out (k_out, B, O * IV * IC) = alpha * sum over the named
    (row, reduced-axis entry) pairs."""
    _chk(data, take)
    k_in = data.shape[0]
    assert data.numel() == k_in * B * O * RED * IV * IC and take.numel() == k_out * n_slots * O * IV
    out = torch.empty((k_out, B, O * IV * IC), device=data.device, dtype=torch.float32)
    with _timed('gather_reduce_rows', (k_in, k_out, n_slots, B, O, RED, IV, IC)):
        check(
            _lib.load().folx_hip_gather_reduce_rows(_stream(), _p(data), _p(take), _p(out), k_in, k_out, n_slots, B, O,
                                                    RED, IV, IC, float(alpha)),
            'gather_reduce_rows',
        )
    return out


def gather_cols(data, table, S_inner=1):
    """out[rb, po, si] = sum_s data[rb, table[po, s], si]: ``data`` (RB, S_in_outer * S_inner),
    ``table`` int32 (S_out_outer, n_slots) on the device -> (RB, S_out_outer * S_inner)."""
    _chk(data, table)
    RB = data.shape[0]
    S_in_outer = data.shape[1] // S_inner
    S_out_outer, n_slots = table.shape
    out = torch.empty((RB, S_out_outer * S_inner), device=data.device, dtype=torch.float32)
    with _timed('gather_cols', (RB, S_in_outer, S_out_outer, n_slots, S_inner)):
        check(
            _lib.load().folx_hip_gather_cols(
                _stream(), _p(data), _p(table), _p(out), RB, S_in_outer, S_out_outer, n_slots, S_inner
            ),
            'gather_cols',
        )
    return out


def scatter_add_rows(data, idx, k_out, B, S_outer, S_inner, out=None):
    """out[idx[r, so], b, so, si] += data[r, b, so, si]; ``out`` = an existing (k_out, B, S)
    row stack to accumulate into (in place), else a zero-filled one is created."""
    _chk(data, idx, out)
    k_in = data.shape[0]
    if out is None:
        out = torch.zeros((k_out, B, S_outer * S_inner), device=data.device, dtype=torch.float32)
    check(
        _lib.load().folx_hip_scatter_add_rows(
            _stream(), _p(data), _p(idx), _p(out), k_in, k_out, B, S_outer, S_inner
        ),
        'scatter_add_rows',
    )
    return out


SMALL_MATRIX_MAX = 32  # largest n (and number of right-hand sides) of the one-matrix-per-wavefront kernels


def slogdet_scaled_supported(n, k_rows):
    return n <= 16 and k_rows <= 4


def slogdet(A, AJ, AL, row_axis=None, factor=None):
    """A (.., n, n), AJ (P, .., n, n), AL (.., n, n) -> sign, logdet (..), jac (P, ..), lap (..).
    ``row_axis`` (an axis of A, default the one before last) names the axis that holds the
    matrix rows; the last axis holds the columns and every other axis is a batch axis, in
    order.  The matrices are read in place, whatever ``row_axis``.  ``factor = (F, FJ, FL,
    index)``: the matrices are ``A * F`` with F of A's shape, FJ (k, ..) sparse rows and
    ``index`` int32 (k, elements per walker) naming their dense rows."""
    _chk(A, AJ, AL)
    n = A.shape[-1]
    P = AJ.shape[0]
    nd = A.dim()
    ra = nd - 2 if row_axis is None else row_axis % nd
    assert ra < nd - 1 and A.shape[ra] == n, 'slogdet needs square matrices'
    outer, mid = tuple(A.shape[:ra]), tuple(A.shape[ra + 1:-1])
    NB = int(np.prod(outer, dtype=np.int64))
    ND = int(np.prod(mid, dtype=np.int64))
    lead = (*outer, *mid)
    sign = torch.empty(lead, device=A.device, dtype=torch.float32)
    ld = torch.empty_like(sign)
    ldj = torch.empty((P, *lead), device=A.device, dtype=torch.float32)
    ldl = torch.empty_like(sign)
    if factor is not None:
        F, FJ, FL, index = factor
        _chk(F, FJ, FL, index)
        assert tuple(F.shape) == tuple(A.shape) and tuple(FJ.shape[1:]) == tuple(A.shape)
        S_w = A.numel() // A.shape[0]
        assert tuple(index.shape) == (FJ.shape[0], S_w) and index.dtype == torch.int32
        with _timed('slogdet_scaled_fwdlap', (NB * ND, n, P, FJ.shape[0])):
            check(
                _lib.load().folx_hip_slogdet_scaled_fwdlap(
                    _stream(), _p(A), _p(AJ), _p(AL), _p(F), _p(FJ), _p(FL), _p(index), _p(sign), _p(ld), _p(ldj),
                    _p(ldl), NB, ND, n, P, n * ND * n, n, ND * n, A.numel(), S_w, FJ.shape[0]
                ),
                'slogdet_scaled_fwdlap',
            )
        return sign, ld, ldj, ldl
    with _timed('slogdet_fwdlap', (NB * ND, n, P)):
        check(
            _lib.load().folx_hip_slogdet_strided_fwdlap(
                _stream(), _p(A), _p(AJ), _p(AL), _p(sign), _p(ld), _p(ldj), _p(ldl), NB, ND, n, P,
                n * ND * n, n, ND * n, A.numel()
            ),
            'slogdet_fwdlap',
        )
    return sign, ld, ldj, ldl


def sparse_slogdet(A, AJ, AL, take, cols, rows, transposed):
    """A (.., n, n), AJ (k, .., n, n) stored rows, AL (.., n, n); int32 device tables take /
    cols (C, rank, width) and rows (C, rank) -> sign, logdet (..), jac (C, ..), lap (..)."""
    _chk(A, AJ, AL, take, cols, rows)
    n = A.shape[-1]
    k = AJ.shape[0]
    C, rank, width = take.shape
    lead = A.shape[:-2]
    NM = int(np.prod(lead, dtype=np.int64)) if len(lead) else 1
    sign = torch.empty(lead, device=A.device, dtype=torch.float32)
    ld = torch.empty_like(sign)
    ldj = torch.empty((C, *lead), device=A.device, dtype=torch.float32)
    ldl = torch.empty_like(sign)
    with _timed('sparse_slogdet_fwdlap', (NM, n, k, C, rank, width)):
        check(
            _lib.load().folx_hip_sparse_slogdet_fwdlap(
                _stream(), _p(A), _p(AJ), _p(AL), _p(take), _p(cols), _p(rows), _p(sign), _p(ld), _p(ldj),
                _p(ldl), NM, n, k, C, rank, width, int(bool(transposed))
            ),
            'sparse_slogdet_fwdlap',
        )
    return sign, ld, ldj, ldl


def inv(A, AJ, AL):
    """A (.., n, n), AJ (P, .., n, n), AL (.., n, n) -> C, C_jac, C_lap of the same shapes."""
    _chk(A, AJ, AL)
    n = A.shape[-1]
    P = AJ.shape[0]
    lead = A.shape[:-2]
    NM = int(np.prod(lead, dtype=np.int64)) if len(lead) else 1
    C, CJ, CL = torch.empty_like(A), torch.empty_like(AJ), torch.empty_like(AL)
    with _timed('inv_fwdlap', (NM, n, P)):
        check(_lib.load().folx_hip_inv_fwdlap(_stream(), _p(A), _p(AJ), _p(AL), _p(C), _p(CJ), _p(CL), NM, n, P),
              'inv_fwdlap')
    return C, CJ, CL


def solve(A, AJ, AL, b, bJ, bL, P):
    """A (.., n, n), b (.., n, m) with equal leading shapes; AJ/AL or bJ/bL may be None for
    a constant operand -> y, y_jac (P, .., n, m), y_lap."""
    _chk(A, AJ, AL, b, bJ, bL)
    n, m = b.shape[-2:]
    lead = A.shape[:-2]
    assert tuple(b.shape[:-2]) == tuple(lead) and A.shape[-1] == n and A.shape[-2] == n
    NM = int(np.prod(lead, dtype=np.int64)) if len(lead) else 1
    y = torch.empty_like(b)
    yJ = torch.empty((P, *b.shape), device=b.device, dtype=torch.float32)
    yL = torch.empty_like(b)
    with _timed('solve_fwdlap', (NM, n, m, P, AJ is not None, bJ is not None)):
        check(
            _lib.load().folx_hip_solve_fwdlap(
                _stream(), _p(A), _p(AJ), _p(AL), _p(b), _p(bJ), _p(bL), _p(y), _p(yJ), _p(yL), NM, n, m, P
            ),
            'solve_fwdlap',
        )
    return y, yJ, yL


def mhsa(q, qj, ql, k, kj, kl, v, vj, vl, mask=None, input_mask=None, edge=None):
    """q/k/v (B, n, H, d) triplets; mask uint8 (B, n); input_mask uint8 (P, B); ``edge`` =
    optional (e, e_jac, e_lap) bias triplet with e (B, n, H, n)."""
    _chk(q, qj, ql, k, kj, kl, v, vj, vl, mask, input_mask)
    B, n, H, d = q.shape
    P = qj.shape[0]
    o, oj, ol = torch.empty_like(q), torch.empty_like(qj), torch.empty_like(q)
    if edge is not None:
        e, ej, el = edge
        _chk(e, ej, el)
        assert tuple(e.shape) == (B, n, H, n) and ej.shape[0] == P
        with _timed('mhsea_fwdlap', (B, n, H, d, P)):
            check(
                _lib.load().folx_hip_mhsea_fwdlap(
                    _stream(), _p(q), _p(qj), _p(ql), _p(k), _p(kj), _p(kl), _p(e), _p(ej), _p(el),
                    _p(v), _p(vj), _p(vl), _p(mask), _p(input_mask), _p(o), _p(oj), _p(ol), B, n, H, d, P,
                ),
                'mhsea_fwdlap',
            )
        return o, oj, ol
    with _timed('mhsa_fwdlap', (B, n, H, d, P)):
        check(
            _lib.load().folx_hip_mhsa_fwdlap(
                _stream(), _p(q), _p(qj), _p(ql), _p(k), _p(kj), _p(kl), _p(v), _p(vj), _p(vl),
                _p(mask), _p(input_mask), _p(o), _p(oj), _p(ol), B, n, H, d, P,
            ),
            'mhsa_fwdlap',
        )
    return o, oj, ol


def mhsa_sparse_supported(n, d, k_rows):
    """Shapes the position-sparse attention kernel is built for."""
    if not (n <= 64 and d <= 64 and d % 4 == 0 and 1 <= k_rows <= 8 and 3 * k_rows * (d // 4) <= 512):
        return False
    # the kernel's LDS footprint (floats), at most 160 KB per workgroup
    lds = (4 * n * (d + 4) + 4 * n * (n + 1) + 4 * (2 * k_rows * (d + 4) + 2 * k_rows * d + 2 * k_rows * n + 2 * k_rows)
           + 5 * n + k_rows * n)
    return 4 * lds <= 160 * 1024


def mhsa_sparse(q, qs, ql, k, ks, kl, v, vs, vl, index, P, all_rows_named):
    """Attention rule for q, k, v (B, n, H, d) whose Jacobians ``*s`` (k_rows, B, n, H, d) are
    sparse by position; ``index`` int32 (k_rows, n) on the device names the dense row of each
    slot.  Returns the triplet with a dense ``(P, B, n, H, d)`` Jacobian."""
    _chk(q, qs, ql, k, ks, kl, v, vs, vl, index)
    B, n, H, d = q.shape
    k_rows = qs.shape[0]
    assert tuple(index.shape) == (k_rows, n) and index.dtype == torch.int32
    o, ol = torch.empty_like(q), torch.empty_like(q)
    oj = (torch.empty if all_rows_named else torch.zeros)((P, B, n, H, d), device=q.device, dtype=torch.float32)
    with _timed('mhsa_sparse_fwdlap', (B, n, H, d, k_rows, P)):
        check(
            _lib.load().folx_hip_mhsa_sparse_fwdlap(
                _stream(), _p(q), _p(qs), _p(ql), _p(k), _p(ks), _p(kl), _p(v), _p(vs), _p(vl),
                _p(index), _p(o), _p(oj), _p(ol), B, n, H, d, k_rows,
            ),
            'mhsa_sparse_fwdlap',
        )
    return o, oj, ol

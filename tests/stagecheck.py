"""Stage-by-stage parity of a whole model on the GPU -- TEST INFRASTRUCTURE.

``with StageCheck() as sc: run the model`` wraps every tensor-level kernel wrapper of
``folx_amd.kernels``: each call still runs the HIP kernel, and in addition the float32 inputs it
was handed are evaluated by the float64 oracle rule of that call (the stand-ins of
``tests/cpu_kernels.py``); the kernel's output must meet the strict bars of
``tests/tolerances.py`` against that reference.  A model at its real width is thereby checked
rule call by rule call on the inputs the HIP path actually produced, independent of how
ill-conditioned the function as a whole is.

Some rules amplify the rounding of their own inputs beyond those bars, whatever computes them:
log|det A| by the condition number of A, an attention row whose terms are larger than their sum.
The allowance for that is measured, not assumed: the oracle rule is evaluated a second time on
inputs perturbed by relative noise of NOISE = 2^-22 (a few float32 roundings), and where the
bar of each output is the strict bar times (1 + the rule's response to that noise in units of the
strict bar): the kernel's own rounding and the conditioning of the rule add up.  The factor
(1.0x for a rule that is well conditioned at its inputs, where the response is a few percent of
the bar) is recorded in ``StageCheck.log`` next to every call.
"""

import numpy as np
import torch

import cpu_kernels as ck
from tolerances import LAP_ATOL, LAP_ATOL_REL, LAP_RTOL, VAL_ATOL_REL, VAL_RTOL

NOISE = 2.0 ** -22  # relative size of the input perturbation that measures a rule's own sensitivity
MAX_ALLOWANCE = 3.0  # largest widening of the bar accepted for a rule that is not a determinant

_TRIPLETS = ('dense', 'dense_act', 'dense_act_parts', 'norm_dense', 'dot_two', 'dot_const', 'exp_envelope', 'layernorm', 'elementwise', 'binary',
             'mul_sparse', 'inv', 'inv_any', 'solve', 'mhsa', 'mhsa_sparse')
_SINGLE = ('rows_affine', 'reduce_sum', 'reduce_max', 'gather_rows', 'gather_reduce_rows', 'gather_cols', 'scatter_add_rows')
_DETS = ('slogdet', 'sparse_slogdet', 'slogdet_any')


def _snap(v):
    """Copy of an argument tree with every tensor cloned (kernels may work in place)."""
    if isinstance(v, torch.Tensor):
        return v.detach().clone()
    if isinstance(v, (list, tuple)):
        return type(v)(_snap(t) for t in v)
    return v


def _np(t):
    return t.detach().cpu().numpy().astype(np.float64)


def _perturb(v, rng):
    """The argument tree with every floating-point tensor multiplied by 1 + NOISE * U(-1, 1)."""
    if isinstance(v, torch.Tensor):
        if not v.dtype.is_floating_point:
            return v
        noise = torch.as_tensor(rng.uniform(-1.0, 1.0, size=tuple(v.shape)), dtype=torch.float64)
        return v.detach().cpu().double() * (1.0 + NOISE * noise)
    if isinstance(v, (list, tuple)):
        return type(v)(_perturb(t, rng) for t in v)
    return v


def _err(got, ref, rtol, atol):
    """max over entries of |got - ref| / (atol + rtol |ref|): <= 1 passes."""
    got, ref = _np(got), _np(ref)
    assert got.shape == ref.shape, (got.shape, ref.shape)
    if ref.size == 0:
        return 0.0
    return float((np.abs(got - ref) / (atol + rtol * np.abs(ref))).max())


def _val_err(got, ref, amp=1.0):
    scale = float(np.abs(_np(ref)).max()) if ref.numel() else 0.0
    return _err(got, ref, VAL_RTOL * amp, (VAL_ATOL_REL * scale + 1e-30) * amp)


def _lap_err(got, ref, amp=1.0):
    scale = float(np.abs(_np(ref)).max()) if ref.numel() else 0.0
    return _err(got, ref, LAP_RTOL * amp, (LAP_ATOL + LAP_ATOL_REL * scale) * amp)


class StageCheck:
    def __init__(self, names=ck.KERNEL_NAMES):
        self.names = tuple(names)
        self.log = []      # (kernel, shape of the first output, worst ratio to the bar, allowance)
        self._orig = {}

    def _wrap(self, name, orig):
        ref_fn = getattr(ck, name)

        def wrapped(*args, **kw):
            # every evaluation gets its own copy of the arguments: a kernel or a stand-in that accumulates into an
            # ``out=`` argument must not be seen by the next evaluation
            a64, kw64 = _snap(args), {k: _snap(v) for k, v in kw.items()}
            out = orig(*args, **kw)
            old = ck.OUT_DTYPE
            ck.OUT_DTYPE = np.float64
            rng = np.random.default_rng(len(self.log))
            try:
                ref = ref_fn(*_snap(a64), **{k: _snap(v) for k, v in kw64.items()})
                per = ref_fn(*_perturb(a64, rng), **{k: _perturb(v, rng) for k, v in kw64.items()})
            finally:
                ck.OUT_DTYPE = old
            if name in _TRIPLETS:
                errs, o, r, q = (_val_err, _val_err, _lap_err), out, ref, per
            elif name in _DETS:
                assert torch.equal(out[0].cpu().double(), ref[0].double()), f'{name}: sign differs from the oracle'
                errs, o, r, q = (_val_err, _val_err, _lap_err), out[1:], ref[1:], per[1:]
            else:
                errs, o, r, q = (_val_err,), (out,), (ref,), (per,)
            # the rule's own response to input noise, in units of the strict bar, widens the bar
            amps = tuple(1.0 + e(qq, rr) for e, qq, rr in zip(errs, q, r))
            parts = tuple(e(oo, rr, a) for e, oo, rr, a in zip(errs, o, r, amps))
            worst, first, amp = max(parts), o[0], max(amps)
            self.log.append((name, tuple(first.shape), worst, amp))
            # only the determinant rules amplify input rounding by more than a few bars (the condition number of the
            # matrix); anywhere else a large allowance means the harness, not the rule, is broken
            assert name in _DETS or amp <= MAX_ALLOWANCE, (
                f'stage {len(self.log)} ({name}, output {tuple(first.shape)}): measured allowance {amp:.1f} exceeds '
                f'{MAX_ALLOWANCE} for a rule that is not a determinant')
            assert worst <= 1.0, (f'stage {len(self.log)} ({name}, output {tuple(first.shape)}): error is {worst:.2f} x the '
                                  f'strict bar (allowance {amp:.1f}; value / Jacobian / Laplacian: '
                                  + ' / '.join(f'{v:.2f}' for v in parts) + ')')
            return out

        return wrapped

    def __enter__(self):
        import folx_amd.kernels as K

        for name in self.names:
            self._orig[name] = getattr(K, name)
            setattr(K, name, self._wrap(name, self._orig[name]))
        return self

    def __exit__(self, *exc):
        import folx_amd.kernels as K

        for name, fn in self._orig.items():
            setattr(K, name, fn)
        self._orig.clear()

    def summary(self):
        """{kernel: (calls, worst ratio to the bar, largest allowance)}"""
        out = {}
        for name, _, worst, amp in self.log:
            c, w, a = out.get(name, (0, 0.0, 1.0))
            out[name] = (c + 1, max(w, worst), max(a, amp))
        return out

"""The generic rule (folx/wrapper.py:73-138) on the GPU: a torch function without a rule of its
own, wrapped and placed between hand-written rules, against the Hessian trace of the whole
composition."""

import numpy as np
import pytest
import torch

from bruteforce import brute_force
from tolerances import assert_lap, assert_val

import folx_amd
from folx_amd import numpy as fnp

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize('thr', [0, 6])
def test_wrapped_torch_function_between_rules(thr):
    rng = np.random.default_rng(46)
    x = rng.normal(size=(5, 4, 3)).astype(np.float32)
    w = rng.normal(size=(3, 2)).astype(np.float32)

    def op(a, b, wc):  # per walker: a (4, 3), b (4,), wc (3, 2)
        return torch.sin(a @ wc) * b[:, None], torch.exp(-b) * a.sum()

    def model(r):
        z, e = fnp.call(op, fnp.tanh(r), fnp.sum(fnp.square(r), axis=-1), w)  # wrapped on the fly
        return fnp.add(fnp.sum(fnp.square(z)), fnp.sum(e))

    out = folx_amd.vmap(folx_amd.forward_laplacian(model, thr))(torch.as_tensor(x).cuda())

    def whole(t):
        z, e = op(torch.tanh(t), (t * t).sum(-1), torch.as_tensor(w, dtype=t.dtype))
        return (z * z).sum() + e.sum()

    by, bJ, bL = brute_force(whole, x.astype(np.float64))
    J = out.jacobian.dense_array
    assert_val(out.x, by, 'value')
    assert_val(J, bJ.reshape(tuple(J.shape)), 'jacobian')
    assert_lap(out.laplacian, bL, 'laplacian')

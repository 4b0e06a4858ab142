"""Parity bars used by the GPU tests (fp32 kernels vs the fp64 oracle on the same inputs).

values / Jacobians : rtol 1e-5
Laplacians         : rtol 1e-4, atol 1e-5
Both get an absolute floor proportional to the largest reference magnitude: an fp32
dot product of K terms carries an absolute error of ~1e-7 * sum|terms|, so entries that
cancel to near zero cannot meet a pure relative bound (the reference's own attention test
adds an atol for the same reason, test/experimental/pallas/test_attention.py:365-386).
"""

import numpy as np

VAL_RTOL = 1e-5
VAL_ATOL_REL = 2e-6   # absolute floor = VAL_ATOL_REL * max|reference|
LAP_RTOL = 1e-4
LAP_ATOL = 1e-5
LAP_ATOL_REL = 1e-5   # plus LAP_ATOL_REL * max|reference| for large-magnitude Laplacians


def _np(t):
    if hasattr(t, 'detach'):
        t = t.detach().cpu().numpy()
    return np.asarray(t, dtype=np.float64)


def assert_val(got, ref, what='value'):
    got, ref = _np(got), _np(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = float(np.abs(ref).max()) if ref.size else 0.0
    np.testing.assert_allclose(got, ref, rtol=VAL_RTOL, atol=VAL_ATOL_REL * scale + 1e-30, err_msg=what)


def assert_lap(got, ref, what='laplacian'):
    got, ref = _np(got), _np(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = float(np.abs(ref).max()) if ref.size else 0.0
    np.testing.assert_allclose(got, ref, rtol=LAP_RTOL, atol=LAP_ATOL + LAP_ATOL_REL * scale, err_msg=what)


def assert_triplet(got, ref, what=''):
    assert_val(got[0], ref[0], what + ' x')
    assert_val(got[1], ref[1], what + ' jacobian')
    assert_lap(got[2], ref[2], what + ' laplacian')

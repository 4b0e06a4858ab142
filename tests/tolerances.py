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


# How often the absolute floors are what lets an entry pass: per kind of bar, entries compared, entries that meet
# the pure relative bound (rtol alone), and the largest |error| / (rtol |ref|) among the others.  Printed at the end
# of a pytest session (tests/conftest.py), and bounded by tests/test_kernels_gpu.py::test_floor_is_used_by_small_entries_only.
FLOOR_STATS = {'value': [0, 0, 0.0], 'laplacian': [0, 0, 0.0]}


def _tally(kind, got, ref, rtol):
    if ref.size == 0:
        return
    diff = np.abs(got - ref)
    pure = diff <= rtol * np.abs(ref)
    st = FLOOR_STATS[kind]
    st[0] += int(ref.size)
    st[1] += int(pure.sum())


def floor_usage(got, ref, rtol):
    """(fraction of entries that need the absolute floor, fraction of max|ref| below which all of them lie)"""
    got, ref = _np(got), _np(ref)
    need = np.abs(got - ref) > rtol * np.abs(ref)
    if not need.any():
        return 0.0, 0.0
    return float(need.mean()), float(np.abs(ref)[need].max() / max(np.abs(ref).max(), 1e-300))


def _np(t):
    if hasattr(t, 'detach'):
        t = t.detach().cpu().numpy()
    return np.asarray(t, dtype=np.float64)


def assert_val(got, ref, what='value'):
    got, ref = _np(got), _np(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = float(np.abs(ref).max()) if ref.size else 0.0
    _tally('value', got, ref, VAL_RTOL)
    np.testing.assert_allclose(got, ref, rtol=VAL_RTOL, atol=VAL_ATOL_REL * scale + 1e-30, err_msg=what)


def assert_lap(got, ref, what='laplacian'):
    got, ref = _np(got), _np(ref)
    assert got.shape == ref.shape, (what, got.shape, ref.shape)
    scale = float(np.abs(ref).max()) if ref.size else 0.0
    _tally('laplacian', got, ref, LAP_RTOL)
    np.testing.assert_allclose(got, ref, rtol=LAP_RTOL, atol=LAP_ATOL + LAP_ATOL_REL * scale, err_msg=what)


def assert_triplet(got, ref, what=''):
    assert_val(got[0], ref[0], what + ' x')
    assert_val(got[1], ref[1], what + ' jacobian')
    assert_lap(got[2], ref[2], what + ' laplacian')

"""Fusion without annotations on the GPU: the benchmark models written with plain calls
(``folx_amd/workloads.py``) launch what the forms with every fusion spelled out
(``tests/annotated_workloads.py``) launch, and return the same bits."""

import pytest
import torch

import annotated_workloads as ann

import folx_amd
from folx_amd import kernels as K
from folx_amd import workloads as wl

pytestmark = pytest.mark.gpu

ANNOTATED = {'mlp_dense': ann.mlp_forward, 'mlp_sparse': ann.mlp_forward, 'ferminet16': ann.ferminet_forward,
             'psiformer32': ann.psiformer_forward, 'psiformer64': ann.psiformer_forward}


def launches(fn, x, thr):
    with K.LaunchTimer() as lt:
        out = folx_amd.vmap(folx_amd.forward_laplacian(fn, thr))(x)
    counts = {}
    for (entry, key), (calls, _ms) in lt.summary().items():
        counts[(entry, key)] = counts.get((entry, key), 0) + calls
    return out, counts


@pytest.mark.parametrize('name', sorted(ANNOTATED))
def test_plain_calls_equal_annotated_form_bit_for_bit(name):
    forward, p, cfg, _, sigma, thr = wl.build(name)
    p = wl.to_device(p, torch.device('cuda'))
    x = wl.sample_inputs(name, 4, seed=3)
    print(f'case plain calls {name}', flush=True)
    got, n_plain = launches(lambda t: forward(p, t), x, thr)
    want, n_ann = launches(lambda t: ANNOTATED[name](p, t), x, thr)
    assert n_plain == n_ann, {k: (n_plain.get(k), n_ann.get(k)) for k in set(n_plain) | set(n_ann) if n_plain.get(k) != n_ann.get(k)}
    assert torch.equal(got.x, want.x) and torch.equal(got.laplacian, want.laplacian)
    assert torch.equal(got.jacobian.dense_array, want.jacobian.dense_array)
    entries = {}
    for (entry, _key), c in n_plain.items():
        entries[entry] = entries.get(entry, 0) + c
    if name.startswith('psiformer'):
        assert entries.get('norm_dense_fwdlap') == 3 * 3 + 4 and entries.get('layernorm_fwdlap') == 1, entries
        assert entries.get('slogdet_scaled_fwdlap' if cfg.n_up <= 16 else 'slogdet_fwdlap') == 2, entries
        assert 'mhsa_sparse_fwdlap' in entries and entries.get('mhsa_fwdlap') == 3, entries
    elif name == 'ferminet16':
        assert entries.get('dense_act_parts_fwdlap', 0) + entries.get('dense_act_fwdlap', 0) >= 6, entries
        assert entries.get('slogdet_scaled_fwdlap') == 2, entries
    else:
        assert entries.get('dense_act_fwdlap') == 10 and 'elementwise_fwdlap' not in entries, entries

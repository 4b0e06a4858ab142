"""``folx_amd.experimental.auto_batched_vmap`` (folx/experimental/vmap.py:14-73) on the GPU: the chunk size comes from
the measured memory of two probe chunks, results are those of ``batched_vmap`` with that chunk size."""

import numpy as np
import pytest
import torch

import folx_amd
from folx_amd import workloads as wl
from folx_amd.experimental import auto_batched_vmap

pytestmark = pytest.mark.gpu


def test_auto_batched_vmap_fits_the_stated_share_of_memory():
    forward, params, cfg, _, sigma, thr = wl.build('mlp_dense')     # 100 nodes x 4 inputs: 400 Jacobian rows per walker
    params = wl.to_device(params, torch.device('cuda'))
    fl = folx_amd.forward_laplacian(lambda r: forward(params, r), thr)
    x = torch.as_tensor(wl.sample_inputs('mlp_dense', 96)).cuda()
    free, _ = torch.cuda.mem_get_info()
    share = 3.0e9 / free                                             # about 3 GB for one chunk
    auto = auto_batched_vmap(fl, max_fraction=share)
    print('auto_batched_vmap on mlp_dense, 96 walkers', flush=True)
    out = auto(x)
    (size,) = auto.chosen.values()
    print(f'chosen chunk: {size} walkers', flush=True)
    assert 1 <= size < 96, size                                      # ~ 0.1 GB per walker: a few tens of walkers fit
    want = folx_amd.batched_vmap(fl, size)(x)
    assert torch.equal(out.x, want.x) and torch.equal(out.laplacian, want.laplacian)
    assert torch.equal(out.jacobian.dense_array, want.jacobian.dense_array)
    # the chosen chunk really stays within the share (the allocator's peak while one chunk runs)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    torch.cuda.reset_peak_memory_stats()
    folx_amd.vmap(fl)(x[:size])
    torch.cuda.synchronize()
    peak = torch.cuda.max_memory_allocated() - before
    assert peak <= 1.1 * share * free, (peak, share * free)
    assert peak >= 0.4 * share * free, (peak, share * free)         # and is not needlessly small
    # second call: no probes, the same choice
    again = auto(x)
    assert torch.equal(again.laplacian, out.laplacian) and len(auto.chosen) == 1


def test_auto_batched_vmap_cap_and_small_batches():
    forward, params, cfg, _, sigma, thr = wl.build('mlp_sparse')
    params = wl.to_device(params, torch.device('cuda'))
    fl = folx_amd.forward_laplacian(lambda r: forward(params, r), thr)
    x = torch.as_tensor(wl.sample_inputs('mlp_sparse', 40)).cuda()
    auto = auto_batched_vmap(fl, max_batch_size=16)
    out = auto(x)
    assert list(auto.chosen.values()) == [16]
    want = folx_amd.batched_vmap(fl, 16)(x)
    assert torch.equal(out.laplacian, want.laplacian)
    few = auto_batched_vmap(fl)                                       # not more walkers than the probes: runs whole
    out = few(x[:12])
    assert list(few.chosen.values()) == [12]
    assert torch.equal(out.laplacian, folx_amd.vmap(fl)(x[:12]).laplacian)

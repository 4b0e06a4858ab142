"""Benchmark of the forward-Laplacian hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload psiformer32]

A step is one full forward Laplacian (value, 96-row Jacobian, Laplacian per walker) of the
PsiFormer-style 32-electron wavefunction over a batch of 4096 synthetic walkers that are
resident in HBM before the timed region starts.  Prints ONE JSON line with walkers/s, the
roofline of the dominant kernel (per-launch durations taken with HIP events on the launch
stream inside the timed region) and the CPU baseline (the numpy oracle on a bounded
sample of the same workload, timed on this host).
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

PEAK_BF16_MFMA_TFLOPS = 2500.0
PEAK_FP32_MFMA_TFLOPS = 157.3  # MI355X dense FP32 matrix peak
PEAK_HBM_GBS = 8000.0

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (two runs, each
# scaled by what the same counter reads for a plain 1 GiB copy: x2.000 and x1.000); the
# figures and the commands are in profiles/psiformer32_forward_laplacian.txt (its HBM table; the fused entries are the
# sums over their launches that the table spells out).
MEASURED_TRAFFIC_BYTES = {
    ('dense_fwdlap', (32768, 96, 256, 256, False)): 6.584e9,
    ('dense_fwdlap', (32768, 96, 256, 256, True)): 9.884e9,
    ('mhsa_fwdlap', (1024, 32, 4, 64, 96)): 13.170e9,
    # fused entry points: the sum over their launches (weights fold, per-position rows, x / lap
    # rows GEMM, Jacobian GEMM, finish)
    ('norm_dense_fwdlap', (None, 32768, 96, 256, 256)): 7.363e9,
    ('norm_dense_fwdlap', ('tanh', 32768, 96, 256, 256)): 7.606e9,
}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=20)
    ap.add_argument('--warmup', type=int, default=5)
    ap.add_argument('--workload', default='psiformer32')
    ap.add_argument('--walkers', type=int, default=0, help='override the batch (0 = the configuration default)')
    ap.add_argument('--chunk', type=int, default=1024, help='walkers per batched_vmap chunk')
    ap.add_argument('--cpu-seconds', type=float, default=20.0, help='budget of the CPU baseline sample')
    ap.add_argument('--no-cpu', action='store_true')
    ap.add_argument('--gemm', choices=('f32', 'bf16x3'), default='f32',
                    help='products of the wide dense rules: FP32 matrix instructions (default) or the exact '
                         'three-piece bf16 split on the bf16 matrix pipe')
    ap.add_argument('--no-split-leg', action='store_true',
                    help='skip the short second measurement with --gemm bf16x3 that a default run appends')
    ap.add_argument('--no-other', action='store_true',
                    help='skip the short measurements of the other workloads that a default run appends')
    ap.add_argument('--streaming-rules', action='store_true',
                    help='instead of a workload: launch every HBM-bound rule at its largest workload shape (ten launches '
                         'each, HIP events) and print one JSON line of achieved TB/s; the command profiles/ traces')
    ap.add_argument('--front-door', choices=('calls', 'torch'), default='calls',
                    help="'torch': the workload's model as plain torch code, traced with torch.fx and evaluated through "
                         'the same rules (folx_amd.forward_laplacian_torch); the default is the model written with '
                         'folx_amd.numpy calls')
    ap.add_argument('--graph', action='store_true',
                    help='replay each chunk as a captured HIP graph (no per-kernel timing, no roofline)')
    ap.add_argument('--calibrate-copy', action='store_true',
                    help='also launch one plain copy (rows_affine, 1 GiB in, 1 GiB out) for scaling HBM counters')
    return ap.parse_args()


def cpu_baseline(workload, budget_s, gpu_out=None, gpu_out_split=None):
    """The numpy oracle (fp32, dense Jacobians) on a bounded sample of the same workload: the first
    n walkers of the batch the GPU was timed on, whose GPU results (``gpu_out``) are compared with
    the oracle's in the same run.  On the first walkers (at most 8) the oracle also runs in float64:
    the GPU's distance from that result stands beside the float32 oracle's own distance from it, so
    that a reader can tell the conditioning of the function from an error of the kernels."""
    from oracle import backend as ob

    from folx_amd import workloads as wl

    forward, p, cfg, _, sigma, _ = wl.build(workload)
    try:
        from threadpoolctl import threadpool_info

        threads = max([i.get('num_threads', 1) for i in threadpool_info()] or [1])
    except Exception:
        threads = 1

    def run(n, dtype=np.float32):
        x = wl.sample_inputs(workload, n, seed=2)  # the first n walkers of the GPU's batch (same seed, row-major draws)
        t0 = time.perf_counter()
        out = forward(p, ob.init_state(x, dtype=dtype), ob)
        dt = time.perf_counter() - t0
        assert np.isfinite(out.lap).all()
        return dt, out

    t1, out = run(1)
    n = int(max(1, min(64, budget_s / max(t1, 1e-3))))
    if n > 1:
        dt, out = run(n)
    else:
        dt = t1
    res = {
        'value': n / dt,
        'unit': 'walkers/s',
        'cores': threads,
        'host_cpu_count': os.cpu_count(),
        'kind': 'port',
        'sample': f'{n} walkers of {workload}, numpy fp32 oracle with dense Jacobians, {dt:.1f} s '
                  f'(BLAS threads {threads} of os.cpu_count() = {os.cpu_count()})',
    }
    if gpu_out is not None:
        # same walkers, GPU path against the CPU oracle: largest difference over the largest reference entry.
        # Both sides are float32; log|det| of the randomly initialised orbital matrices amplifies their
        # rounding, which is what these figures show -- `against_fp64` below separates the two, and the
        # parity bars are enforced stage by stage in tests/.
        rel = lambda g, r, m: float(np.abs(g[..., :m].astype(np.float64) - r).max() / max(np.abs(r).max(), 1e-30))
        parts = lambda o, m: (np.asarray(o.x, dtype=np.float64)[None, :m],
                              np.asarray(o.J, dtype=np.float64).reshape(o.J.shape[0], -1)[:, :m],
                              np.asarray(o.lap, dtype=np.float64)[None, :m])

        def against(triplet, ref, m):
            gx, gJ, gl = triplet
            rx, rJ, rl = ref
            return {'value': rel(gx[None], rx, m), 'jacobian': rel(gJ, rJ, m), 'laplacian': rel(gl[None], rl, m),
                    'walkers': m}

        res['gpu_vs_oracle_max_rel'] = against(gpu_out, parts(out, n), n)
        if gpu_out_split is not None:  # the run with the bf16x3 products, same walkers
            res['bf16x3_vs_oracle_max_rel'] = against(gpu_out_split, parts(out, n), n)
        m = min(n, 8)
        _, out64 = run(m, np.float64)
        ref64 = parts(out64, m)
        o32 = parts(out, m)
        res['against_fp64'] = {
            'what': f'first {m} walkers: max |result - float64 oracle| / max |float64 oracle|; the float32 oracle\'s own '
                    'distance is the rounding floor of this function in float32',
            'gpu_vs_fp64': against(gpu_out, ref64, m),
            'oracle_fp32_vs_fp64': against((o32[0][0], o32[1], o32[2][0]), ref64, m),
        }
        if gpu_out_split is not None:
            res['against_fp64']['bf16x3_vs_fp64'] = against(gpu_out_split, ref64, m)
    return res


def describe(cfg):
    if hasattr(cfg, 'n_nodes'):
        return (f'node-wise MLP, {cfg.n_nodes} nodes x {cfg.in_dim} inputs, {cfg.n_hidden} x [Dense({cfg.width}) + SiLU] '
                f'+ Dense(1), summed')
    if hasattr(cfg, 'n_heads'):
        return (f'PsiFormer-style, {cfg.n_elec} electrons, {cfg.n_nuc} nuclei, {cfg.n_layers} layers x '
                f'{cfg.n_heads} heads x {cfg.head_dim}, width {cfg.width}, {cfg.n_det} determinants')
    return (f'FermiNet-style, {cfg.n_elec} electrons, {cfg.n_nuc} nuclei, {cfg.n_layers} layers, one-electron '
            f'width {cfg.w1}, two-electron width {cfg.w2}, {cfg.n_det} determinants')


def roofline_of(dname, dkey, dn, dms, gemm):
    """Roofline record of one entry point and shape: algorithmic flops or bytes of the rule (the per-unit
    figures of the kernels' own headers) over the average duration of its launches."""
    avg_s = dms / dn * 1e-3
    mfma = lambda flops, kernel: {'bound': 'mfma', 'achieved': flops / avg_s / 1e12, 'peak': PEAK_FP32_MFMA_TFLOPS,
                                  'unit': 'TFLOP/s', 'frac': flops / avg_s / 1e12 / PEAK_FP32_MFMA_TFLOPS,
                                  'traffic': MEASURED_TRAFFIC_BYTES.get((dname, dkey)), 'kernel': kernel,
                                  'launches': dn, 'avg_launch_ms': dms / dn}
    hbm = lambda nbytes, kernel: {'bound': 'hbm', 'achieved': nbytes / avg_s / 1e9, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                                  'frac': nbytes / avg_s / 1e9 / PEAK_HBM_GBS, 'traffic': None, 'kernel': kernel,
                                  'launches': dn, 'avg_launch_ms': dms / dn}
    if dname == 'dense_fwdlap':
        R, P, Kd, N, has_res = dkey
        if N == 1:  # matrix-vector form
            return hbm(4.0 * (P + 2) * R * (Kd + 1), f'dense_n1 kernels R={R} P={P} K={Kd}')
        kern = (('dense_split_kernel' if gemm == 'bf16x3' and N > 128 else 'dense_dma_kernel')
                if Kd % 16 == 0 and N % 4 == 0 else 'dense_kernel')
        return mfma(2.0 * (P + 2) * R * Kd * N, kern + f' R={R} P={P} K={Kd} N={N} residual={has_res}')
    if dname == 'mhsa_fwdlap':
        Bc, n, H, d, P = dkey
        return mfma((7.0 * P + 6) * 2 * n * n * d * Bc * H, f'mhsa_kernel B={Bc} n={n} H={H} d={d} P={P}')
    if dname == 'norm_dense_fwdlap' or (dname == 'dense_act_fwdlap' and dkey[4] > 128):
        # the wide fused rules: one GEMM over the Jacobian rows (tiles cut across Jacobian rows)
        # plus short launches for the x / lap rows; the events bracket the whole entry point
        act, R, P, Kd, N = dkey
        norm = dname == 'norm_dense_fwdlap'
        return mfma(2.0 * (P + 2) * R * Kd * N,
                    f'dense_wide_kernel<{"true" if norm else "false"}, {"false" if act is None else "true"}, '
                    f'{"32, false" if norm else "16 | 32, parts"}, {"true" if gemm == "bf16x3" else "false"}> '
                    f'+ the short launches of its entry point '
                    f'({dname}: x / lap rows GEMM, finish; with LayerNorm also weight fold and per-position rows), '
                    f'act={act} R={R} P={P} K={Kd} N={N}')
    if dname == 'dense_act_fwdlap':
        act, R, P, Kd, N = dkey
        r = hbm(4.0 * ((P + 2) * R * (Kd + N) + Kd * N), f'dense_act_kernel {act} R={R} P={P} K={Kd} N={N}')
        r['mfma_tflops'] = 2.0 * (P + 2) * R * Kd * N / avg_s / 1e12
        r['mfma_frac'] = r['mfma_tflops'] / PEAK_FP32_MFMA_TFLOPS
        return r
    if dname == 'elementwise_fwdlap':
        name, S, P = dkey
        return hbm(8.0 * (P + 2) * S, f'elementwise_kernel<{name}> S={S} P={P}')
    if dname == 'layernorm_fwdlap':
        R, F, P = dkey
        return hbm(8.0 * (P + 2) * R * F, f'layernorm_kernel R={R} F={F} P={P}')
    if dname == 'reduce_sum':
        rows, outer, red, inner = dkey
        return hbm(4.0 * rows * outer * (red + 1) * inner, f'reduce kernels rows={rows} outer={outer} red={red} inner={inner}')
    if dname == 'mhsa_sparse_fwdlap':
        Bc, n, H, d, k, P = dkey
        return hbm(4.0 * n * d * (P + 3 * k + 8) * Bc * H, f'mhsa_sparse_kernel B={Bc} n={n} H={H} d={d} k={k} P={P}')
    if dname in ('slogdet_fwdlap', 'slogdet_scaled_fwdlap'):
        NM, n, P = dkey[:3]
        k = dkey[3] if len(dkey) > 3 else -2
        return hbm(4.0 * NM * n * n * ((P + 2) + (k + 2)), f'slogdet kernels NM={NM} n={n} P={P}')
    return {'bound': 'hbm', 'achieved': None, 'peak': PEAK_HBM_GBS, 'unit': 'GB/s', 'frac': None,
            'traffic': None, 'kernel': f'{dname} {dkey}', 'launches': dn, 'avg_launch_ms': dms / dn}


def measure(workload, steps, warmup, walkers=0, chunk=1024, gemm='f32', graph=False, calibrate_copy=False,
            front_door='calls'):
    """Times ``steps`` steps of one workload after ``warmup`` untimed ones (inputs resident on the device, host clock
    around device synchronisations) and finds the entry point with the largest total time, whose launches carry HIP
    events on the launch stream inside the timed region.  Returns the pieces of the output line."""
    import torch

    import folx_amd
    from folx_amd import kernels as K
    from folx_amd import workloads as wl

    forward, params_np, cfg, B, sigma, thr = wl.build(workload)
    if walkers:
        B = walkers
    dev = torch.device('cuda', 0)
    params = wl.to_device(params_np, dev)
    x = torch.as_tensor(wl.sample_inputs(workload, B, seed=2)).to(dev)
    if front_door == 'torch':
        # the same model as plain torch code, traced once (torch.fx) and evaluated through the rules
        from folx_amd import torch_namespace as txp

        fl = folx_amd.forward_laplacian_torch(lambda r: forward(params_np, r, xp=txp), thr)
    else:
        fl = folx_amd.forward_laplacian(lambda r: forward(params, r), thr)
    step = folx_amd.batched_vmap(folx_amd.jit(folx_amd.vmap(fl)) if graph else fl, chunk)

    for _ in range(warmup):
        out = step(x)
    torch.cuda.synchronize()
    if calibrate_copy:
        n = 1 << 28  # 2^28 floats = 1 GiB read + 1 GiB written by rows_affine_kernel
        src = torch.empty(n, device=dev, dtype=torch.float32).fill_(1.0)
        K.rows_affine(src, 1, (n,), (n,), None, None, 1.0, 0.0)
        torch.cuda.synchronize()
        del src

    # One untimed step with every entry point bracketed by events: the per-kernel breakdown, and
    # which entry point dominates.  In the timed region only that one carries events (an event pair
    # per launch costs host time and keeps neighbouring kernels from overlapping, which a
    # workload of many short launches would pay for in its headline figure).
    # (Taken from the second of two such steps: the first timed launch of a process can carry a one-off stall of
    # tens of milliseconds, which would land on whatever entry point happens to come first.)
    for _ in range(2):
        with K.LaunchTimer() as lt_all:
            out = step(x)
        summ_all = lt_all.summary()
    dominant = max(summ_all.items(), key=lambda kv: kv[1][1])[0][0] if summ_all else None
    with K.LaunchTimer(only=() if dominant is None else (dominant,)) as lt:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            out = step(x)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    assert torch.isfinite(out.x).all() and torch.isfinite(out.laplacian).all()
    summ = lt.summary()
    roof = None
    if summ:
        (dname, dkey), (dn, dms) = max(summ.items(), key=lambda kv: kv[1][1])
        roof = roofline_of(dname, dkey, dn, dms, gemm)
        roof['entry_point'] = dname
        roof['share_of_gpu_time'] = dms / steps / max(sum(ms for (_n, ms) in summ_all.values()), 1e-30)
    per_kernel = {}
    for (name, key), (n, ms) in summ_all.items():
        per_kernel[name] = per_kernel.get(name, 0.0) + ms
    return {'B': B, 'cfg': cfg, 'thr': thr, 'out': out, 'x': x, 'step': step, 'dt': dt, 'roof': roof,
            'per_kernel': per_kernel, 'graph_mode': not summ}


# the other BASELINE.json configurations, measured briefly after the headline: (steps, warm-up steps, chunk)
GRAPH_REPLAY_TOO = ('mlp_dense', 'mlp_sparse', 'ferminet16')
OTHER_WORKLOADS = {'mlp_dense': (20, 5, 1024), 'mlp_sparse': (20, 5, 1024), 'ferminet16': (8, 4, 1024),
                   'psiformer64': (2, 1, 1024)}


def streaming_rules():
    """Every HBM-bound rule at the largest shape the benchmark workloads give it (a chunk of 1024 walkers): achieved
    rate = the rule's algorithmic bytes (the per-unit figures of the kernels' headers) over the mean duration of ten
    launches, HIP events on the launch stream.  One JSON line; `rocprofv3 --kernel-trace --stats` of this command gives
    the same durations kernel by kernel."""
    import torch

    from folx_amd import kernels as K

    dev = torch.device('cuda', 0)
    g = torch.Generator(device='cuda').manual_seed(0)
    rn = lambda *s: torch.randn(*s, device=dev, generator=g)  # noqa: E731
    table = []

    def run(name, kernel, fn, nbytes, reps=10):
        for _ in range(2):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        table.append({'rule': name, 'kernel': kernel, 'avg_us': 1e3 * ms, 'algorithmic_GB': nbytes / 1e9,
                      'TB_per_s': nbytes / ms / 1e9, 'frac_of_8TBps': nbytes / ms / 1e9 / (PEAK_HBM_GBS / 1e3)})

    n = 1 << 28
    src = rn(n)
    run('plain copy of 1 GiB (calibration of the HBM counters)', 'rows_affine_v4_kernel',
        lambda: K.rows_affine(src, 1, (n,), (n,), None, None, 1.0, 0.0), 8.0 * n)
    d2 = rn(n)
    run('sum of two row stacks, 1 GiB each', 'rows_affine_v4_kernel',
        lambda: K.rows_affine(src, 1, (n,), (n,), None, d2, 1.0, 1.0), 12.0 * n)
    del src, d2
    R, F, P = 32768, 256, 96                        # 1024 walkers x 32 electrons, width 256, dense Jacobian
    x, J, L = rn(R, F), rn(P, R, F), rn(R, F)
    run('tanh, P = 96 dense rows', 'elementwise_kernel', lambda: K.elementwise('tanh', x, J, L), 8.0 * (P + 2) * R * F)
    gam, bet = rn(F), rn(F)
    run('LayerNorm, P = 96 dense rows', 'layernorm_kernel<1, false>', lambda: K.layernorm(x, J, L, gam, bet, 1e-5),
        8.0 * (P + 2) * R * F)
    J3 = rn(3, R, F)
    run('LayerNorm, k = 3 sparse rows (first layer)', 'layernorm_kernel<1, true>',
        lambda: K.layernorm(x, J3, L, gam, bet, 1e-5), 8.0 * 5 * R * F, reps=30)
    run('tanh, k = 3 sparse rows', 'elementwise_kernel', lambda: K.elementwise('tanh', x, J3, L), 8.0 * 5 * R * F, reps=30)
    J2 = rn(P, R, F)
    run('product of two triplets, P = 96', 'binary_kernel<0>', lambda: K.binary('mul', x, J, L, x, J2, L),
        12.0 * (P + 2) * R * F)
    del J2
    idx = torch.arange(3 * 32, device=dev, dtype=torch.int32).reshape(3, 32)
    idxf = idx[:, :, None].expand(3, 32, 256).reshape(3, -1).contiguous()
    v = lambda t, lead: t.view(*lead, 1024, -1)  # noqa: E731
    run('dense x sparse product, P = 96, k = 3', 'mul_sparse_kernel<4, 4>',
        lambda: K.mul_sparse(v(x, ()), v(J, (P,)), v(L, ()), v(x, ()), v(J3, (3,)), v(L, ()), idxf),
        4.0 * (2 * P + 3 + 6) * R * F)
    del J
    data = rn(3, 1024, 32 * 256)
    take = torch.full((96, 1, 32), -1, device=dev, dtype=torch.int32)
    for so_ in range(32):
        for r in range(3):
            take[3 * so_ + r, 0, so_] = r
    run('sparse -> dense hand-off, k = 3 rows to 96', 'gather_rows_flat_kernel<4>',
        lambda: K.gather_rows(data, take, 96, 1, 1024, 32, 256), 4.0 * (3 + 96) * 1024 * 32 * 256)
    out = rn(96, 1024, 32 * 256)
    run('sparse skip connection added in place, k = 3 into 96 rows', 'scatter_add_rows_kernel<4>',
        lambda: K.scatter_add_rows(data, idx, 96, 1024, 32, 256, out=out), 4.0 * 3 * 3 * 1024 * 32 * 256, reps=30)
    del out, data
    inp = rn(1, 49152, 16, 256)
    run('sum over 16 electrons of a (48 x 1024, 16, 256) stack', 'reduce_mid_v4_kernel',
        lambda: K.reduce_sum(inp, 1, 49152, 16, 256), 4.0 * 49152 * 17 * 256, reps=30)
    del inp
    A, AJ, AL = rn(16384, 16, 16), rn(96, 16384, 16, 16), rn(16384, 16, 16)
    run('slogdet, 16384 matrices 16 x 16, P = 96', 'slogdet16_kernel<16, false, 4>', lambda: K.slogdet(A, AJ, AL),
        4.0 * 98 * 256 * 16384)
    A, AJ, AL = rn(16384, 8, 8), rn(48, 16384, 8, 8), rn(16384, 8, 8)
    run('slogdet, 16384 matrices 8 x 8, P = 48', 'slogdet16_kernel<8, false, 4>', lambda: K.slogdet(A, AJ, AL),
        4.0 * 50 * 64 * 16384, reps=30)
    A, AJ, AL = rn(16384, 32, 32), rn(192, 16384, 32, 32), rn(16384, 32, 32)
    run('slogdet, 16384 matrices 32 x 32, P = 192', 'slogdet32_kernel', lambda: K.slogdet(A, AJ, AL),
        4.0 * 194 * 1024 * 16384, reps=5)
    table[-1]['mfma_TFLOP_per_s'] = 2.0 * 192 * 32768 * 16384 / (table[-1]['avg_us'] * 1e-6) / 1e12
    del A, AJ, AL
    B, n_, H, d, k, Pd = 1024, 32, 4, 64, 3, 96
    q, qs, ql = rn(B, n_, H, d) / 8, rn(k, B, n_, H, d) / 8, rn(B, n_, H, d) / 8
    ix = torch.arange(k * n_, device=dev, dtype=torch.int32).reshape(n_, k).t().contiguous()
    run('attention on position-sparse rows, k = 3 -> P = 96', 'mhsa_sparse_kernel',
        lambda: K.mhsa_sparse(q, qs, ql, q, qs, ql, q, qs, ql, ix, Pd, True), 4.0 * n_ * d * (Pd + 3 * k + 8) * B * H)
    print(json.dumps({'metric': 'achieved HBM rate of the streaming rules at their largest workload shapes',
                      'peak_TB_per_s': PEAK_HBM_GBS / 1e3, 'rules': table}))


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get('WORLD_SIZE', '1')) != 1:
        print('bench.py measures one GPU: walkers are independent, every GPU would run this same '
              'path on its share of the batch; run with --gpus 1', file=sys.stderr)
        sys.exit(2)

    import torch

    from folx_amd import kernels as K

    torch.cuda.set_device(0)
    K.set_gemm_mode(args.gemm)
    if args.streaming_rules:
        streaming_rules()
        return
    m = measure(args.workload, args.steps, args.warmup, args.walkers, args.chunk, args.gemm, args.graph,
                args.calibrate_copy, args.front_door)
    B, cfg, thr, out, x, step, dt, roof = (m[k] for k in ('B', 'cfg', 'thr', 'out', 'x', 'step', 'dt', 'roof'))
    ms_per_step = 1e3 * dt / args.steps
    value = B * args.steps / dt
    if m['graph_mode']:
        line = {'metric': 'walkers/s of full forward Laplacian at 1 GPU', 'value': value, 'unit': 'walkers/s',
                'n_gpus': 1, 'steps': args.steps, 'warmup': args.warmup, 'ms_per_step': ms_per_step,
                'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None, 'dtype': 'f32',
                'data': 'synthetic', 'config': {'workload': f'{args.workload}: {describe(cfg)}', 'walkers': B,
                                                'chunk': args.chunk, 'mode': 'hip graph replay'},
                'roofline': None}
        print(json.dumps(line))
        return

    line = {
        'metric': 'walkers/s of full forward Laplacian at 1 GPU',
        'value': value,
        'unit': 'walkers/s',
        'n_gpus': 1,
        'steps': args.steps,
        'warmup': args.warmup,
        'ms_per_step': ms_per_step,
        'higher_is_better': True,
        'scaling': 'weak',
        'vs_baseline': None,
        'dtype': 'f32',
        'data': 'synthetic',
        'config': {
            'workload': f'{args.workload}: {describe(cfg)}, ForwardLaplacianOperator({thr})',
            'walkers': B,
            'chunk': args.chunk,
            'jacobian_rows': int(out.jacobian.dense_array.shape[0]),
            'gemm': args.gemm,
            'front_door': args.front_door,
        },
        'roofline': roof,
        # from the one untimed step in which every entry point carried events
        'kernel_ms_per_step': {k: v for k, v in sorted(m['per_kernel'].items(), key=lambda kv: -kv[1])},
    }
    if roof is not None and roof.get('traffic') is not None:
        roof['traffic_source'] = ('profiles/psiformer32_forward_laplacian.txt, table "HBM counters": rocprofv3 --pmc FETCH_SIZE / '
                                  'WRITE_SIZE of this command in earlier runs, summed over the launches of the entry point '
                                  '(counters cannot be read inside the timed run)')
    if args.gemm == 'bf16x3' and roof is not None and roof['bound'] == 'mfma' and 'mhsa' not in roof['kernel']:
        # six bf16 piece products per fp32 product: the matrix pipe's bf16 peak over six
        roof['peak'] = PEAK_BF16_MFMA_TFLOPS / 6.0
        roof['frac'] = roof['achieved'] / roof['peak']
        roof['peak_note'] = 'bf16 dense peak 2500 TFLOP/s / 6 piece products per fp32 product'
    if args.gemm == 'f32' and not args.no_split_leg and not args.graph:
        # the same step with the products of the wide dense rules on the bf16 pipe (three exact bf16
        # pieces per operand): reported beside the headline, never as `value`
        K.set_gemm_mode('bf16x3')
        out2 = None
        try:
            out2 = step(x)
            torch.cuda.synchronize()
            n2 = max(1, min(args.steps, 5))
            t0 = time.perf_counter()
            for _ in range(n2):
                out2 = step(x)
            torch.cuda.synchronize()
            dt2 = time.perf_counter() - t0
            line['bf16x3_products'] = {
                'value': B * n2 / dt2, 'unit': 'walkers/s', 'steps': n2, 'ms_per_step': 1e3 * dt2 / n2,
                'how': 'FOLX_AMD_GEMM=bf16x3 / folx_hip_set_gemm_mode(1); fp32 inputs, outputs and accumulators'}
        except Exception as e:  # the side measurement must not take the headline line down with it
            out2 = None
            line['bf16x3_products'] = {'error': f'{type(e).__name__}: {e}'}
        finally:
            K.set_gemm_mode('f32')
    else:
        out2 = None
    if (not args.no_other and args.gemm == 'f32' and args.workload == 'psiformer32' and not args.walkers
            and args.front_door == 'calls' and not args.graph):
        # the same model as plain torch code through the traced front door (torch.fx graph evaluated through the
        # rules): reported beside the headline, never as `value`
        try:
            import folx_amd
            from folx_amd import torch_namespace as txp
            from folx_amd import workloads as wl

            forward, params_np = wl.build(args.workload)[:2]
            traced = folx_amd.batched_vmap(
                folx_amd.forward_laplacian_torch(lambda r: forward(params_np, r, xp=txp), thr), args.chunk)
            out3 = traced(x)
            torch.cuda.synchronize()
            n3 = max(1, min(args.steps, 3))
            t0 = time.perf_counter()
            for _ in range(n3):
                out3 = traced(x)
            torch.cuda.synchronize()
            dt3 = time.perf_counter() - t0
            rel = (out3.laplacian - out.laplacian).abs() / out.laplacian.abs().clamp_min(1e-30)
            line['traced_torch_front_door'] = {
                'value': B * n3 / dt3, 'unit': 'walkers/s', 'steps': n3, 'ms_per_step': 1e3 * dt3 / n3,
                # per walker |difference| / |Laplacian| against the headline run (a different order of float32
                # operations; the few walkers with near-singular orbital matrices carry the tail)
                'laplacian_relative_difference_to_headline': {'median': float(rel.median()),
                                                              'p99': float(rel.quantile(0.99))},
                'how': 'folx_amd.forward_laplacian_torch: the model as plain torch code, traced once with torch.fx, '
                       'every equation evaluated through the rule registry'}
            del out3, traced
        except Exception as e:  # the side measurement must not take the headline line down with it
            line['traced_torch_front_door'] = {'error': f'{type(e).__name__}: {e}'}
    if not args.no_other and args.gemm == 'f32' and args.workload == 'psiformer32' and not args.walkers:
        # the other configurations of the benchmark suite, a few steps each: walkers/s, the entry point with
        # the largest total time and its roofline fraction.  The headline stays the line's `value`.
        others = {}
        for name, (k_steps, k_warm, k_chunk) in OTHER_WORKLOADS.items():
            try:
                o = measure(name, k_steps, k_warm, 0, k_chunk)
                r = o['roof'] or {}
                others[name] = {
                    'value': o['B'] * k_steps / o['dt'], 'unit': 'walkers/s', 'walkers': o['B'], 'steps': k_steps,
                    'warmup': k_warm, 'ms_per_step': 1e3 * o['dt'] / k_steps,
                    'workload': f"{describe(o['cfg'])}, ForwardLaplacianOperator({o['thr']})",
                    'dominant': {k: r.get(k) for k in ('entry_point', 'kernel', 'bound', 'achieved', 'unit', 'frac',
                                                       'avg_launch_ms', 'share_of_gpu_time', 'mfma_frac') if k in r},
                }
                del o
                if name in GRAPH_REPLAY_TOO:
                    # the reference runs under jax.jit; its counterpart here is the replay of a captured HIP graph,
                    # which takes the host's rule dispatch out of a step made of many short launches
                    o = measure(name, k_steps, k_warm, 0, k_chunk, graph=True)
                    others[name]['hip_graph_replay'] = {'value': o['B'] * k_steps / o['dt'], 'unit': 'walkers/s',
                                                        'ms_per_step': 1e3 * o['dt'] / k_steps}
                    del o
            except Exception as e:  # a side measurement must not take the headline line down with it
                others.setdefault(name, {})['error'] = f'{type(e).__name__}: {e}'
            torch.cuda.empty_cache()
        line['other_workloads'] = others
    if not args.no_cpu:
        host = lambda o: (o.x.cpu().numpy(), o.jacobian.dense_array.reshape(-1, B).cpu().numpy(),  # noqa: E731
                          o.laplacian.cpu().numpy())
        gpu_out = host(out) if tuple(out.x.shape) == (B,) else None
        gpu_out2 = host(out2) if out2 is not None and gpu_out is not None else None
        line['cpu_baseline'] = cpu_baseline(args.workload, args.cpu_seconds, gpu_out, gpu_out2)
        if 'bf16x3_vs_oracle_max_rel' in line['cpu_baseline']:  # same walkers, same oracle run as the headline's figures
            line.setdefault('bf16x3_products', {})['gpu_vs_oracle_max_rel'] = line['cpu_baseline'].pop('bf16x3_vs_oracle_max_rel')
    del out2
    # the reference itself (JAX on the host cores) can only be timed where jax is installed
    import importlib.util

    if importlib.util.find_spec('jax') is None:
        line['reference_jax_cpu'] = 'unavailable on this host (jax is not installed)'
        print('reference JAX-CPU: unavailable on this host', file=sys.stderr)
    print(json.dumps(line))


if __name__ == '__main__':
    main()

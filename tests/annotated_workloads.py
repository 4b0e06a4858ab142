"""The benchmark models with every fusion spelled out through keyword arguments of
``folx_amd.numpy`` (``act=``, ``residual=``, ``row_slice=``, ``window=``, ``factor=``, ``row_axis=``) --
TEST INFRASTRUCTURE.  ``folx_amd/workloads.py`` writes the same models with plain calls only and
relies on the front end to find the fusions; ``tests/test_plain_calls*.py`` require both forms to
issue the same kernel launches and to return the same bits."""

import numpy as np

from folx_amd.workloads import electron_nuclear_features


def mlp_forward(params, x, xp=None):
    if xp is None:
        from folx_amd import numpy as xp
    for W, b in params[:-1]:
        x = xp.dot(x, W, b, act='silu')
    W, b = params[-1]
    return xp.sum(xp.dot(x, W, b))


def psiformer_forward(p, r, xp=None):
    """log|psi(r)| for one walker; r (n_elec, 3)."""
    if xp is None:
        from folx_amd import numpy as xp
    cfg = p.cfg
    n, H, dh = cfg.n_elec, cfg.n_heads, cfg.head_dim
    d, dist = electron_nuclear_features(xp, r, p.nuclei)
    feats = xp.concatenate([xp.reshape(d, (n, 3 * cfg.n_nuc)), dist, p.spin], axis=-1)
    h = xp.dot(feats, p.w_in)
    for L in p.layers:
        # the LayerNorms are only consumed by matrix products, which take them into their own
        # rule where they can (dense Jacobians): the normalised Jacobian is then never written
        hn = xp.layer_norm(h, L['ln1_g'], L['ln1_b'], cfg.ln_eps)
        q = xp.reshape(xp.dot(hn, L['w_q']), (n, H, dh))
        k = xp.reshape(xp.dot(hn, L['w_k']), (n, H, dh))
        v = xp.reshape(xp.dot(hn, L['w_v']), (n, H, dh))
        att = xp.multi_head_self_attention(q, k, v)
        h = xp.dot(xp.reshape(att, (n, H * dh)), L['w_o'], None, residual=h)
        hn = xp.layer_norm(h, L['ln2_g'], L['ln2_b'], cfg.ln_eps)
        h = xp.dot(xp.dot(hn, L['w_1'], L['b_1'], act='tanh'), L['w_2'], L['b_2'], residual=h)
    logdets, signs = [], []
    for s, (lo, hi) in enumerate([(0, cfg.n_up), (cfg.n_up, n)]):
        m = hi - lo
        if m == 0:
            continue
        orb = xp.dot(h, p.w_orb[s], row_slice=(lo, hi))  # (m, n_det * m), spin block read in place
        env = xp.exp_envelope(xp.getitem(dist, (slice(lo, hi),)), p.env_sigma[s], p.env_pi[s])  # (m, n_det * m)
        # (electron, determinant, orbital): the matrices are read in place, rows on axis 0, and
        # multiplied by their envelopes while they are loaded
        if cfg.orb_shift:
            shift = (cfg.orb_shift * np.eye(m, dtype=np.float32))[:, None, :]
            mats = xp.add(xp.multiply(xp.reshape(orb, (m, cfg.n_det, m)), xp.reshape(env, (m, cfg.n_det, m))), shift)
            sg, ld = xp.slogdet(mats, row_axis=0)
        else:
            sg, ld = xp.slogdet(xp.reshape(orb, (m, cfg.n_det, m)), row_axis=0,
                                factor=xp.reshape(env, (m, cfg.n_det, m)))
        logdets.append(ld), signs.append(sg)
    total = logdets[0] if len(logdets) == 1 else xp.add(logdets[0], logdets[1])
    sign = signs[0] if len(signs) == 1 else xp.multiply(signs[0], signs[1])
    logpsi, _ = xp.logsumexp(total, axis=0, b=sign)
    return logpsi


def ferminet_forward(p, r, xp=None):
    """log|psi(r)| for one walker; r (n_elec, 3)."""
    if xp is None:
        from folx_amd import numpy as xp
    cfg = p.cfg
    n, nu = cfg.n_elec, cfg.n_up
    d, dist = electron_nuclear_features(xp, r, p.nuclei)
    h = xp.concatenate([xp.reshape(d, (n, 3 * cfg.n_nuc)), dist], axis=-1)  # (n, 4 nuc)
    # pair features; the distance of an electron to itself is regularised as in FermiNet:
    # |r_ij + eye| * (1 - eye), so the square root is never taken at zero
    rij = xp.subtract(xp.expand_dims(r, 1), xp.expand_dims(r, 0))  # (n, n, 3)
    r2 = xp.add(xp.sum(xp.square(rij), axis=-1), p.eye)
    rn = xp.multiply(xp.sqrt(r2), 1.0 - p.eye)
    g = xp.concatenate([rij, xp.expand_dims(rn, 2)], axis=-1)  # (n, n, 4)

    def spin_means(t, axis_len):
        # means over the electrons of one spin: the slices are summed where they lie
        up = xp.mean(t, axis=0, window=(0, nu)) if nu > 0 else None
        dn = xp.mean(t, axis=0, window=(nu, n)) if n - nu > 0 else None
        return up, dn

    for li, L in enumerate(p.layers):
        hu, hd = spin_means(h, n)  # (d1,) each
        # means over the second electron of every pair: (n, d2)
        gu = xp.mean(g, axis=1, window=(0, nu))
        gd = xp.mean(g, axis=1, window=(nu, n))
        d1 = h.shape[-1]
        # the feature vector is only consumed by the product below, which reads it part by
        # part where it can: neither the broadcasts nor the concatenation are then formed
        parts = [h, xp.broadcast_to(hu, (n, d1)), xp.broadcast_to(hd, (n, d1)), gu, gd]
        f = xp.concatenate(parts, axis=-1)
        if L['v'].shape[1] == d1:  # residual layer: the skip connection is added in the product's epilogue
            h = xp.dot(f, L['v'], L['b'], act='tanh', residual=h)
        else:
            h = xp.dot(f, L['v'], L['b'], act='tanh')
        if 'w' in L:
            if L['w'].shape[0] == L['w'].shape[1]:  # residual layer of the pair stream: skip connection in the epilogue
                g = xp.dot(g, L['w'], L['c'], act='tanh', residual=g)
            else:
                g = xp.dot(g, L['w'], L['c'], act='tanh')
    logdets, signs = [], []
    for s, (lo, hi) in enumerate([(0, nu), (nu, n)]):
        m = hi - lo
        if m == 0:
            continue
        orb = xp.dot(h, p.w_orb[s], row_slice=(lo, hi))
        env = xp.exp_envelope(xp.getitem(dist, (slice(lo, hi),)), p.env_sigma[s], p.env_pi[s])
        if cfg.orb_shift:
            shift = (cfg.orb_shift * np.eye(m, dtype=np.float32))[:, None, :]
            mats = xp.add(xp.multiply(xp.reshape(orb, (m, cfg.n_det, m)), xp.reshape(env, (m, cfg.n_det, m))), shift)
            sg, ld = xp.slogdet(mats, row_axis=0)
        else:
            sg, ld = xp.slogdet(xp.reshape(orb, (m, cfg.n_det, m)), row_axis=0,
                                factor=xp.reshape(env, (m, cfg.n_det, m)))
        logdets.append(ld), signs.append(sg)
    total = logdets[0] if len(logdets) == 1 else xp.add(logdets[0], logdets[1])
    sign = signs[0] if len(signs) == 1 else xp.multiply(signs[0], signs[1])
    logpsi, _ = xp.logsumexp(total, axis=0, b=sign)
    return logpsi

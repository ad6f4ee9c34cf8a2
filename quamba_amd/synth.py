"""Seeded synthetic inputs shaped like the quantized Mamba mixer's tensors (numpy, CPU).

Activations are N(0,1) with 1% of the channels scaled 20x (outlier channels), quantised to int8
with one symmetric absmax scale per tensor; dt is drawn so that softplus(dt + dt_bias) lies in
[1e-3, 1e-1]; A_log = log(U[1,16]); D = 1.  One generator per tensor name, so changing one shape
does not perturb the other tensors.
"""
import zlib

import numpy as np


def rng_for(seed, name):
    return np.random.default_rng([seed, zlib.crc32(name.encode())])


def quantize_absmax(x, n_bits=8):
    """Symmetric per-tensor quantisation: returns (int8 array, float32 scale)."""
    qmax = 2 ** (n_bits - 1) - 1
    s = np.float32(max(float(np.abs(x).max()), 1e-5) / qmax)
    q = np.clip(np.rint(x / s), -qmax - 1, qmax).astype(np.int8)
    return q, s


def activations(shape, channel_axis, seed, name, outliers=True):
    """float32 N(0,1) with ceil(1%) outlier channels along channel_axis scaled by 20."""
    g = rng_for(seed, name)
    x = g.standard_normal(shape, dtype=np.float32)
    if outliers:
        nch = shape[channel_axis]
        k = max(1, int(np.ceil(0.01 * nch)))
        idx = g.permutation(nch)[:k]
        sl = [slice(None)] * len(shape)
        sl[channel_axis] = idx
        x[tuple(sl)] *= 20.0
    return x


def softplus(x):
    return np.where(x <= 20.0, np.log1p(np.exp(np.minimum(x, 20.0))), x)


def inv_softplus(y):
    return y + np.log(-np.expm1(-y))


def conv_weights(dim, width, seed, bias=True):
    """int8 depthwise conv taps and bias with their per-tensor scales."""
    g = rng_for(seed, "conv_w")
    w = g.uniform(-0.5, 0.5, (dim, width)).astype(np.float32)
    qw, sw = quantize_absmax(w)
    if not bias:
        return qw, sw, None, np.float32(1.0)
    b = rng_for(seed, "conv_b").uniform(-0.5, 0.5, (dim,)).astype(np.float32)
    qb, sb = quantize_absmax(b)
    return qw, sw, qb, sb


def conv_output_scale(qx, sx, qw, sw, qb, sb, silu=True):
    """Output scale = max |act(conv(x))| / 127 from a float64 evaluation of the dequantised conv."""
    B, D, L = qx.shape
    k = qw.shape[1]
    x = qx.astype(np.float64) * float(sx)
    w = qw.astype(np.float64) * float(sw)
    acc = np.zeros((B, D, L))
    for j in range(k):
        shift = k - 1 - j
        if shift < L:
            acc[:, :, shift:] += w[None, :, j, None] * x[:, :, :L - shift]
    if qb is not None:
        acc += (qb.astype(np.float64) * float(sb))[None, :, None]
    if silu:
        acc = acc / (1.0 + np.exp(-acc))
    return np.float32(max(float(np.abs(acc).max()), 1e-5) / 127.0)


def conv_float(qx, sx, qw, sw, qb, sb, silu=True):
    """float64 evaluation of the dequantised depthwise causal conv (+SiLU): (B, D, L)."""
    B, D, L = qx.shape
    k = qw.shape[1]
    x = qx.astype(np.float64) * float(sx)
    w = qw.astype(np.float64) * float(sw)
    acc = np.zeros((B, D, L))
    for j in range(k):
        shift = k - 1 - j
        if shift < L:
            acc[:, :, shift:] += w[None, :, j, None] * x[:, :, :L - shift]
    if qb is not None:
        acc += (qb.astype(np.float64) * float(sb))[None, :, None]
    if silu:
        acc = acc / (1.0 + np.exp(-acc))
    return acc


def mamba2_conv_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, width=4, seed=1234, grouped=True,
                       nhead_groups=4, ndim_groups=4, bias=True):
    """Synthetic inputs of the Mamba2 xBC conv: int8 xBC (batch, dim, seqlen) with separate per-tensor
    scales for the x, B and C parts, int8 taps and bias quantised per part, and output scales taken
    from a float64 evaluation: per (ssd group, head group, dim group) for x when ``grouped`` (uneven
    cumulative end-index tables), per ssd group for B and C, else one scale per part."""
    x_dim, bc = nheads * headdim, ngroups * dstate
    dim = x_dim + 2 * bc
    parts = [(0, x_dim), (x_dim, x_dim + bc), (x_dim + bc, dim)]
    act = activations((batch, dim, seqlen), 1, seed, "xBC")
    qx = np.empty((batch, dim, seqlen), np.int8)
    s_in = []
    for lo, hi in parts:
        q, s = quantize_absmax(act[:, lo:hi])
        qx[:, lo:hi] = q
        s_in.append(s)
    w = rng_for(seed, "conv2_w").uniform(-0.5, 0.5, (dim, width)).astype(np.float32)
    b = rng_for(seed, "conv2_b").uniform(-0.5, 0.5, (dim,)).astype(np.float32)
    qw = np.empty((dim, width), np.int8)
    qb = np.empty((dim,), np.int8) if bias else None
    s_w, s_b = [], []
    for lo, hi in parts:
        q, s = quantize_absmax(w[lo:hi])
        qw[lo:hi] = q
        s_w.append(s)
        if bias:
            q, s = quantize_absmax(b[lo:hi])
            qb[lo:hi] = q
            s_b.append(s)
        else:
            s_b.append(None)
    ref = np.empty((batch, dim, seqlen))
    for i, (lo, hi) in enumerate(parts):
        ref[:, lo:hi] = conv_float(qx[:, lo:hi], s_in[i], qw[lo:hi], s_w[i], qb[lo:hi] if bias else None,
                                   s_b[i] if bias else 1.0)
    amax = lambda a: np.float32(max(float(np.abs(a).max()), 1e-5) / 127.0)
    out = dict(xBC=qx, weight=qw, bias=qb, scales_in=s_in, scales_w=s_w, scales_b=s_b, x_dim=x_dim, bc=bc, dim=dim,
               ref=ref)
    if not grouped:
        out.update(x_out_scales=np.array([amax(ref[:, :x_dim])], np.float32),
                   B_out_scales=np.array([amax(ref[:, x_dim:x_dim + bc])], np.float32),
                   C_out_scales=np.array([amax(ref[:, x_dim + bc:])], np.float32),
                   x_head_group_range=None, x_dim_group_range=None)
        return out
    heads_per_group = nheads // ngroups
    g = rng_for(seed, "conv2_groups")

    def cuts(total, n):
        # n uneven pieces: cumulative end indices, last == total
        if n == 1:
            return np.array([total], np.int32)
        inner = np.sort(g.choice(np.arange(1, total), size=n - 1, replace=False))
        return np.concatenate([inner, [total]]).astype(np.int32)

    nhg = min(nhead_groups, heads_per_group)
    ndg = min(ndim_groups, headdim)
    hr = np.stack([cuts(heads_per_group, nhg) for _ in range(ngroups)])
    dr = np.stack([np.stack([cuts(headdim, ndg) for _ in range(nhg)]) for _ in range(ngroups)])
    xs = np.empty((ngroups, nhg, ndg), np.float32)
    rx = ref[:, :x_dim].reshape(batch, ngroups, heads_per_group, headdim, seqlen)
    for gi in range(ngroups):
        h0 = 0
        for hg in range(nhg):
            d0 = 0
            for dg in range(ndg):
                xs[gi, hg, dg] = amax(rx[:, gi, h0:hr[gi, hg], d0:dr[gi, hg, dg]])
                d0 = dr[gi, hg, dg]
            h0 = hr[gi, hg]
    Bs = np.array([amax(ref[:, x_dim + gi * dstate:x_dim + (gi + 1) * dstate]) for gi in range(ngroups)], np.float32)
    Cs = np.array([amax(ref[:, x_dim + bc + gi * dstate:x_dim + bc + (gi + 1) * dstate]) for gi in range(ngroups)],
                  np.float32)
    out.update(x_out_scales=xs, B_out_scales=Bs, C_out_scales=Cs, x_head_group_range=hr, x_dim_group_range=dr)
    return out


def mamba1_scan_inputs(batch, seqlen, dim, dstate, seed=1234, with_z=True):
    """Quantised inputs of the Mamba1 selective scan: dict of int8 arrays and float32 scales.

    u, dt, z: (batch, dim, seqlen); B, C: (batch, dstate, seqlen); A_log: (dim, dstate);
    D, dt_bias: (dim).
    """
    out = {}
    u = activations((batch, dim, seqlen), 1, seed, "u")
    out["u"], out["s_u"] = quantize_absmax(u)
    g = rng_for(seed, "dt")
    dt_target = np.exp(g.uniform(np.log(1e-3), np.log(1e-1), (batch, dim, seqlen))).astype(np.float32)
    dt_init = np.exp(rng_for(seed, "dt_bias").uniform(np.log(1e-3), np.log(1e-1), (dim,))).astype(np.float32)
    dt_bias = inv_softplus(dt_init.astype(np.float64)).astype(np.float32)
    dt_raw = (inv_softplus(dt_target.astype(np.float64)) - dt_bias[None, :, None]).astype(np.float32)
    out["dt"], out["s_dt"] = quantize_absmax(dt_raw)
    out["dt_bias"], out["s_db"] = quantize_absmax(dt_bias)
    A_log = np.log(rng_for(seed, "A").uniform(1.0, 16.0, (dim, dstate))).astype(np.float32)
    out["A_log"], out["s_A"] = quantize_absmax(A_log)
    out["D"], out["s_D"] = quantize_absmax(np.ones((dim,), np.float32))
    Bm = activations((batch, dstate, seqlen), 1, seed, "B", outliers=False)
    Cm = activations((batch, dstate, seqlen), 1, seed, "C", outliers=False)
    out["B"], out["s_B"] = quantize_absmax(Bm)
    out["C"], out["s_C"] = quantize_absmax(Cm)
    if with_z:
        z = activations((batch, dim, seqlen), 1, seed, "z")
        out["z"], out["s_z"] = quantize_absmax(z)
    else:
        out["z"], out["s_z"] = None, np.float32(0.0)
    return out


def linear_weights(out_features, in_features, seed, name="w", per_channel=True):
    """int8 weights (N,K) ~ N(0, 1/sqrt(K)) with per-output-channel (or per-tensor) scales."""
    g = rng_for(seed, name)
    w = (g.standard_normal((out_features, in_features), dtype=np.float32) / np.sqrt(in_features)).astype(np.float32)
    if per_channel:
        s = np.maximum(np.abs(w).max(axis=1), 1e-5).astype(np.float32) / np.float32(127.0)
        q = np.clip(np.rint(w / s[:, None]), -128, 127).astype(np.int8)
        return q, s.astype(np.float32), w
    q, s = quantize_absmax(w)
    return q, np.array([s], np.float32), w


def mamba2_ssd_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, seed=1234, grouped=False,
                      nhead_groups=4, ndim_groups=4, with_z=False):
    """Quantised inputs of the Mamba2 SSD chunk scan.

    x (batch, seqlen, nheads, headdim), dt (batch, seqlen, nheads), B, C (batch, seqlen, ngroups, dstate)
    int8; A_log, D (nheads) int8; dt_bias (nheads) fp16.  With ``grouped`` the x scale is per
    (ssd group, head group, dim group) with equal-sized groups and B/C scales per ssd group.
    """
    out = {}
    x = activations((batch, seqlen, nheads, headdim), 2, seed, "x2")
    g = rng_for(seed, "dt2")
    dt_target = np.exp(g.uniform(np.log(1e-3), np.log(1e-1), (batch, seqlen, nheads))).astype(np.float32)
    dt_init = np.exp(rng_for(seed, "dt_bias2").uniform(np.log(1e-3), np.log(1e-1), (nheads,))).astype(np.float32)
    dt_bias = inv_softplus(dt_init.astype(np.float64)).astype(np.float16)
    dt_raw = (inv_softplus(dt_target.astype(np.float64)) - dt_bias.astype(np.float64)[None, None, :]).astype(np.float32)
    out["dt"], out["s_dt"] = quantize_absmax(dt_raw)
    out["dt_bias"] = dt_bias
    out["dt_f32"] = dt_target
    A_log = rng_for(seed, "A2").uniform(0.0, np.log(16.0), (nheads,)).astype(np.float32)      # A = -exp(U[0, log 16])
    out["A_log"], out["s_A"] = quantize_absmax(A_log)
    out["D"], out["s_D"] = quantize_absmax(np.ones((nheads,), np.float32))
    Bm = activations((batch, seqlen, ngroups, dstate), 3, seed, "B2", outliers=False)
    Cm = activations((batch, seqlen, ngroups, dstate), 3, seed, "C2", outliers=False)
    if not grouped:
        out["x"], sx = quantize_absmax(x)
        out["x_scale"] = np.array([sx], np.float32)
        out["B"], sB = quantize_absmax(Bm)
        out["C"], sC = quantize_absmax(Cm)
        out["s_B"], out["s_C"] = np.array([sB], np.float32), np.array([sC], np.float32)
        out["head_range"] = out["dim_range"] = None
    else:
        hpg = nheads // ngroups
        assert hpg % nhead_groups == 0 and headdim % ndim_groups == 0
        hs, ds = hpg // nhead_groups, headdim // ndim_groups
        out["head_range"] = np.tile(np.arange(1, nhead_groups + 1, dtype=np.int32) * hs, (ngroups, 1))
        out["dim_range"] = np.tile(np.arange(1, ndim_groups + 1, dtype=np.int32) * ds, (ngroups, nhead_groups, 1))
        qx = np.empty(x.shape, np.int8)
        xs = np.empty((ngroups, nhead_groups, ndim_groups), np.float32)
        for gi in range(ngroups):
            for hg in range(nhead_groups):
                for dg in range(ndim_groups):
                    sl = (slice(None), slice(None), slice(gi * hpg + hg * hs, gi * hpg + (hg + 1) * hs),
                          slice(dg * ds, (dg + 1) * ds))
                    qx[sl], xs[gi, hg, dg] = quantize_absmax(x[sl])
        out["x"], out["x_scale"] = qx, xs
        qB, qC = np.empty(Bm.shape, np.int8), np.empty(Cm.shape, np.int8)
        sB, sC = np.empty(ngroups, np.float32), np.empty(ngroups, np.float32)
        for gi in range(ngroups):
            qB[:, :, gi], sB[gi] = quantize_absmax(Bm[:, :, gi])
            qC[:, :, gi], sC[gi] = quantize_absmax(Cm[:, :, gi])
        out["B"], out["C"], out["s_B"], out["s_C"] = qB, qC, sB, sC
    if with_z:
        out["z"], out["s_z"] = quantize_absmax(activations((batch, seqlen, nheads, headdim), 2, seed, "z2"))
    else:
        out["z"], out["s_z"] = None, np.float32(0.0)
    return out

"""Independent float64 / integer forms of the same computations, written from the mathematics
(not from the kernels), used only to pin oracle/qoracle.c.  TEST INFRASTRUCTURE ONLY."""
import numpy as np


def softplus(x):
    x = np.asarray(x, np.float64)
    return np.where(x <= 20.0, np.log1p(np.exp(np.minimum(x, 20.0))), x)


def silu(x):
    return x / (1.0 + np.exp(-x))


def selective_scan(u, delta, A, B, C, D=None, z=None, delta_bias=None, delta_softplus=True, h0=None):
    """Textbook Mamba1 selective scan in float64 on real-valued inputs.

    u, delta, z: (batch, dim, L); A: (dim, N) (already -exp(A_log)); B, C: (batch, N, L); D,
    delta_bias: (dim).  h_t = exp(delta_t A) h_{t-1} + delta_t B_t u_t;  y_t = C_t . h_t + D u_t;
    y_t *= silu(z_t).  Returns (y (batch, L, dim), last state (batch, dim, N)).
    """
    u = np.asarray(u, np.float64)
    delta = np.asarray(delta, np.float64)
    batch, dim, L = u.shape
    N = A.shape[1]
    if delta_bias is not None:
        delta = delta + np.asarray(delta_bias, np.float64)[None, :, None]
    if delta_softplus:
        delta = softplus(delta)
    h = np.zeros((batch, dim, N)) if h0 is None else np.array(h0, np.float64)
    y = np.zeros((batch, L, dim))
    for t in range(L):
        dA = np.exp(delta[:, :, t, None] * A[None])                       # (batch, dim, N)
        dBu = delta[:, :, t, None] * B[:, None, :, t] * u[:, :, t, None]
        h = dA * h + dBu
        yt = np.einsum("bdn,bn->bd", h, C[:, :, t])
        if D is not None:
            yt = yt + np.asarray(D, np.float64)[None] * u[:, :, t]
        if z is not None:
            yt = yt * silu(np.asarray(z, np.float64)[:, :, t])
        y[:, t] = yt
    return y, h


def ssd_recurrence(x, dt, A, B, C, D=None, z=None):
    """Textbook Mamba2 (scalar A per head) recurrence in float64 on real-valued inputs.

    x: (batch, L, H, P); dt: (batch, L, H) already processed; A: (H) negative; B, C: (batch, L, G, N);
    D: (H) or (H, P).  h_t = exp(dt_t A) h_{t-1} + dt_t x_t B_t^T;  y_t = h_t C_t + D x_t.
    Returns (y (batch, L, H, P), final state (batch, H, P, N)).
    """
    x = np.asarray(x, np.float64)
    batch, L, H, P = x.shape
    G, N = B.shape[2], B.shape[3]
    rep = H // G
    h = np.zeros((batch, H, P, N))
    y = np.zeros((batch, L, H, P))
    for t in range(L):
        dA = np.exp(dt[:, t] * A[None])                                   # (batch, H)
        Bt = np.repeat(B[:, t], rep, axis=1)                              # (batch, H, N)
        Ct = np.repeat(C[:, t], rep, axis=1)
        h = dA[:, :, None, None] * h + (dt[:, t, :, None] * x[:, t])[..., None] * Bt[:, :, None, :]
        yt = np.einsum("bhpn,bhn->bhp", h, Ct)
        if D is not None:
            Dv = np.asarray(D, np.float64)
            yt = yt + x[:, t] * (Dv[None, :, None] if Dv.ndim == 1 else Dv[None])
        if z is not None:
            yt = yt * silu(np.asarray(z, np.float64)[:, t])
        y[:, t] = yt
    return y, h

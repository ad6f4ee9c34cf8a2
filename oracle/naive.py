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

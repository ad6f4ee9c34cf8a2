"""What an fp16 rounding tie can do to one output of the SSD chunk scan (test helper, CPU only).

Both the kernels and the oracle round the same operands to fp16 before a product - the entering state P_c[p, n] and
the weights w[m, k] = CB[m, k] exp(dA_m - dA_k) dt_k - and accumulate in fp32.  Where the fp32 value of such an operand
lies on a rounding tie the last bit of exp (or the order of an fp32 sum) decides which neighbour it becomes, and the
product moves by one fp16 ulp of that operand.  For one output y[t, p] this module recomputes the sum in float64 from
the oracle's stage tensors and returns the interval the output can reach when every fp16-rounded operand is nudged by
at most one fp16 ulp either way.  An output of the kernels that misses the oracle's value by more than the test's bar
must lie inside that interval; an indexing mistake (a dropped or misplaced term) moves it by a whole term, far outside.
"""
import numpy as np

ULP16 = 2.0 ** -10          # one fp16 ulp is at most this fraction of the value


def _f16(a):
    return np.asarray(a, np.float32).astype(np.float16).astype(np.float64)


def output_interval(ref, t, p, *, chunk, x_codes, x_scale_p, C_codes, s_C, D_weight=0.0):
    """Interval of y[t, p] for a single (batch, head) problem.

    ref: oracle.ssd_fwd(..., stages=True) of that problem (batch 1, one head, one group);
    x_codes int8 (L, P); x_scale_p: scale of channel p; C_codes int8 (L, N); D_weight = D_scale * q_D of the channel.
    Returns (lo, hi, y64)."""
    Q = chunk
    c, m = divmod(int(t), Q)
    dA = ref["dA_cumsum"][0, 0, c].astype(np.float64)
    dtv = ref["dt"][0, 0, c].astype(np.float64)
    L = x_codes.shape[0]
    k = np.arange(0, m + 1)
    k = k[c * Q + k < L]
    # term 2: the causal part of the chunk
    w = ref["CB"][0, c, 0, m, k].astype(np.float64) * np.exp(np.minimum(dA[m] - dA[k], 0.0)) * dtv[k]
    xh = _f16(np.float32(x_scale_p) * x_codes[c * Q + k, p].astype(np.float32))
    t2 = _f16(w) * xh
    # term 1: the state entering the chunk
    t1 = np.zeros(1)
    if c > 0:
        Ch = _f16(np.float32(s_C) * C_codes[t].astype(np.float32))
        t1 = np.exp(dA[m]) * Ch * _f16(ref["prev_states"][0, c, 0, p])
    skip = D_weight * float(np.float32(x_scale_p) * np.float32(x_codes[t, p]))
    y64 = float(t1.sum() + t2.sum() + skip)
    slack = ULP16 * float(np.abs(t1).sum() + np.abs(t2).sum())
    return y64 - slack, y64 + slack, y64

"""CPU oracle for the quantized Mamba mixer path (numpy in, numpy out).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by bench.py's
cpu_baseline leg, never by quamba_amd/.  The arithmetic lives in qoracle.c (a C restatement of
the reference kernels, each function citing the file:line it follows); this module builds it
with gcc and wraps it with ctypes.  ``naive`` holds independent float64 / integer forms used to
pin the restatement itself.

Parity status: every function below is pinned by the checks in tests/test_oracle_*.py (closed
forms, float64 brute force, integer matmul, library routines).  The reference holds no golden
vectors for this path and its kernels (CUDA / Triton-CUDA) cannot be built or run here, so the
exact low-order bits of the reference binaries are not a target.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqoracle.so")
_lib = None

_i8p = np.ctypeslib.ndpointer(np.int8, flags="C_CONTIGUOUS")
_f32p = np.ctypeslib.ndpointer(np.float32, flags="C_CONTIGUOUS")
_i32p = np.ctypeslib.ndpointer(np.int32, flags="C_CONTIGUOUS")


def build(force=False):
    src = os.path.join(_HERE, "qoracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(src) > os.path.getmtime(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE, "-B", "libqoracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.qo_expf.restype = C.c_float
        _lib.qo_expf.argtypes = [C.c_float]
        _lib.qo_sat8_half_away.argtypes = [C.c_float]
        _lib.qo_sat8_rne.argtypes = [C.c_float]
    return _lib


def _opt(a, dtype=np.int8):
    if a is None:
        return None
    return np.ascontiguousarray(a, dtype=dtype).ctypes.data_as(C.c_void_p)


def _req(a, dtype=np.int8):
    a = np.ascontiguousarray(a, dtype=dtype)
    return a, a.ctypes.data_as(C.c_void_p)


def _f(v):
    return C.c_float(float(np.float32(v)))


def expf(x):
    """The deterministic exp of the int8-output ops, elementwise on a float32 array."""
    x = np.asarray(x, dtype=np.float32)
    out = np.empty_like(x)
    l = lib()
    flat_in, flat_out = x.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = l.qo_expf(C.c_float(float(flat_in[i])))
    return out


def conv1d_fwd(x, weight, bias, s_x, s_w, s_b, s_out, silu=True, tapwise=False):
    """x int8 (B,D,L), weight int8 (D,k), bias int8 (D) or None -> int8 (B,D,L)."""
    x, xp = _req(x)
    weight, wp = _req(weight)
    B, D, L = x.shape
    out = np.empty_like(x)
    keep = _opt(bias)
    lib().qo_conv1d_fwd(xp, wp, keep, out.ctypes.data_as(C.c_void_p), B, D, L, weight.shape[1],
                        _f(s_x), _f(s_w), _f(s_b), _f(s_out), int(silu), int(tapwise))
    return out


def conv1d_update(x, state, weight, bias, s_x, s_w, s_b, s_out, silu=True):
    """x int8 (B,D); state int8 (B,D,S) with S in {k, k-1}.  Returns (out int8 (B,D), new state)."""
    x, xp = _req(x)
    weight, wp = _req(weight)
    state = np.array(state, dtype=np.int8, order="C", copy=True)
    B, D = x.shape
    out = np.empty_like(x)
    lib().qo_conv1d_update(xp, state.ctypes.data_as(C.c_void_p), wp, _opt(bias), out.ctypes.data_as(C.c_void_p),
                           B, D, weight.shape[1], state.shape[2], _f(s_x), _f(s_w), _f(s_b), _f(s_out), int(silu))
    return out, state


def quamba2_conv_channel_scales(x_dim, x_headdim, d_state, n_groups, scales_in, scales_w, scales_b,
                                x_out_scales, B_out_scales, C_out_scales, x_head_group_range=None,
                                x_dim_group_range=None):
    """Per-channel (s_in, s_bias, s_out) of the concatenated [x | B | C] channels, resolved the way
    quamba2_conv1d_fwd_kernel.cuh:147-212 does: an x channel belongs to ssd group c // (x_dim / n_groups),
    head (c % group_size) // headdim, position c % headdim; the head group is the first whose
    cumulative end index exceeds the head, the dim group likewise; B/C channel c belongs to ssd group
    c // d_state.  scales_in / scales_w / scales_b are (x, B, C) triples of floats."""
    bc = d_state * n_groups
    dim = x_dim + 2 * bc
    s_in = np.empty(dim, np.float32)
    s_bias = np.empty(dim, np.float32)
    s_out = np.zeros(dim, np.float32)
    grouped = x_head_group_range is not None and x_dim_group_range is not None
    xs = np.asarray(x_out_scales, np.float32)
    Bs = np.asarray(B_out_scales, np.float32).reshape(-1)
    Cs = np.asarray(C_out_scales, np.float32).reshape(-1)
    for c in range(dim):
        part = 0 if c < x_dim else (1 if c < x_dim + bc else 2)
        s_in[c] = np.float32(scales_w[part]) * np.float32(scales_in[part])
        s_bias[c] = np.float32(scales_b[part]) if scales_b[part] is not None else np.float32(0)
        if part == 0:
            if not grouped:
                s_out[c] = xs.reshape(-1)[0]
                continue
            group_size = x_dim // n_groups
            g, head, d = c // group_size, (c % group_size) // x_headdim, c % x_headdim
            hr = np.asarray(x_head_group_range)[g]
            dr = np.asarray(x_dim_group_range)[g]
            h_start = 0
            for hg in range(hr.shape[0]):
                if h_start <= head < hr[hg]:
                    d_start = 0
                    for dg in range(dr.shape[1]):
                        if d_start <= d < dr[hg, dg]:
                            s_out[c] = xs.reshape(n_groups, hr.shape[0], dr.shape[1])[g, hg, dg]
                            break
                        d_start = dr[hg, dg]
                    break
                h_start = hr[hg]
        else:
            local = c - x_dim - (bc if part == 2 else 0)
            src = Bs if part == 1 else Cs
            s_out[c] = src[local // d_state] if grouped else src[0]
    return s_in, s_bias, s_out


def quamba2_conv1d_fwd(xBC, weight, bias, s_in, s_bias, s_out, x_dim, bc, silu=True):
    """xBC int8 (B, dim, L) -> (x int8 (B, x_dim, L), B int8 (B, bc, L), C int8 (B, bc, L)) with the
    per-channel scales of quamba2_conv_channel_scales."""
    xBC, xp = _req(xBC)
    weight, wp = _req(weight)
    batch, dim, L = xBC.shape
    out = np.empty_like(xBC)
    s_in, s_bias, s_out = (np.ascontiguousarray(a, np.float32) for a in (s_in, s_bias, s_out))
    fp = lambda a: a.ctypes.data_as(C.c_void_p)
    lib().qo_conv1d_fwd_perchannel(xp, wp, _opt(bias), fp(out), batch, dim, L, weight.shape[1],
                                   fp(s_in), fp(s_bias), fp(s_out), int(silu))
    return out[:, :x_dim], out[:, x_dim:x_dim + bc], out[:, x_dim + bc:]


def quamba2_conv1d_update(xBC, state, weight, bias, s_in, s_bias, s_out, x_dim, bc, silu=True):
    """xBC int8 (B, dim); state int8 (B, dim, S), S in {k, k-1}.  Returns (x, B, C, new state)."""
    xBC, xp = _req(xBC)
    weight, wp = _req(weight)
    state = np.array(state, dtype=np.int8, order="C", copy=True)
    batch, dim = xBC.shape
    out = np.empty_like(xBC)
    s_in, s_bias, s_out = (np.ascontiguousarray(a, np.float32) for a in (s_in, s_bias, s_out))
    fp = lambda a: a.ctypes.data_as(C.c_void_p)
    lib().qo_conv1d_update_perchannel(xp, fp(state), wp, _opt(bias), fp(out), batch, dim, weight.shape[1],
                                      state.shape[2], fp(s_in), fp(s_bias), fp(s_out), int(silu))
    return out[:, :x_dim], out[:, x_dim:x_dim + bc], out[:, x_dim + bc:], state


def sscan_fwd(u, delta, A_log, B, C_, D=None, delta_bias=None, z=None, *, s_u, s_delta, s_A, s_B, s_C,
              s_D=0.0, s_db=0.0, s_z=0.0, s_state=1.0, softplus=True):
    """u/delta/z int8 (B,D,L); A_log int8 (D,N); B,C int8 (B,G,N,L) or (B,N,L).
    Returns (y float32 (B,L,D) before the fp16 cast, last state int8 (B,D,N), last state fp32)."""
    u, up = _req(u)
    delta, dp = _req(delta)
    A_log, ap = _req(A_log)
    B = np.asarray(B)
    C_ = np.asarray(C_)
    if B.ndim == 3:
        B = B[:, None]
    if C_.ndim == 3:
        C_ = C_[:, None]
    B, bp = _req(B)
    C_, cp = _req(C_)
    batch, dim, L = u.shape
    N = A_log.shape[1]
    G = B.shape[1]
    y = np.empty((batch, L, dim), np.float32)
    st8 = np.empty((batch, dim, N), np.int8)
    st32 = np.empty((batch, dim, N), np.float32)
    lib().qo_sscan_fwd(up, dp, ap, bp, cp, _opt(D), _opt(delta_bias), _opt(z),
                       _f(s_u), _f(s_delta), _f(s_A), _f(s_B), _f(s_C), _f(s_D), _f(s_db), _f(s_z), _f(s_state),
                       batch, dim, L, N, G, int(softplus),
                       y.ctypes.data_as(C.c_void_p), st8.ctypes.data_as(C.c_void_p), st32.ctypes.data_as(C.c_void_p))
    return y, st8, st32


def sscan_update(state, x, dt, A_log, B, C_, D=None, dt_bias=None, z=None, *, s_x, s_dt, s_A, s_B, s_C,
                 s_D=0.0, s_db=0.0, s_z=0.0, s_state=1.0, softplus=True):
    """state int8 or float32 (B,D,N) (not modified; the new state is returned); x, dt, z int8 (B,D);
    B, C int8 (B,N).  Returns (y float32 (B,D), new state)."""
    x, xp = _req(x)
    dt, dp = _req(dt)
    A_log, ap = _req(A_log)
    B, bp = _req(B)
    C_, cp = _req(C_)
    batch, dim = x.shape
    N = A_log.shape[1]
    y = np.empty((batch, dim), np.float32)
    state = np.array(state, order="C", copy=True)
    if state.dtype == np.float32:
        s8, s32 = None, state.ctypes.data_as(C.c_void_p)
    else:
        assert state.dtype == np.int8
        s8, s32 = state.ctypes.data_as(C.c_void_p), None
    lib().qo_sscan_update(s8, s32, xp, dp, ap, bp, cp, _opt(D), _opt(dt_bias), _opt(z),
                          _f(s_x), _f(s_dt), _f(s_A), _f(s_B), _f(s_C), _f(s_D), _f(s_db), _f(s_z), _f(s_state),
                          batch, dim, N, int(softplus), y.ctypes.data_as(C.c_void_p))
    return y, state


def ssm_update_heads(state, x, dt, A_log, B, C_, D=None, dt_bias=None, z=None, *, x_scale, s_dt, s_A, s_B, s_C,
                     s_D=0.0, s_z=0.0, state_scale=1.0, head_range=None, dim_range=None, softplus=True):
    """One recurrence step in the layout with heads (Mamba2, and Mamba1 as one head).
    state int8 or float32 (B,H,P,N) (not modified; the new state is returned); x, z int8 (B,H,P);
    dt int8 broadcastable to (B,H,P); A_log int8 broadcastable to (H,P,N); B, C int8 (B,G,N); D int8
    broadcastable to (H,P); dt_bias float broadcastable to (H,P), holding the value that is added to dt.
    Without head_range / dim_range: x_scale, s_B, s_C, state_scale scalars (requantisation factor 1e2);
    with them: x_scale (G,hg,dg), s_B / s_C (G), state_scale (G,hg,dg,N), int32 cumulative end indices
    head_range (G,hg) and dim_range (G,hg,dg) (factor 1e6).  Returns (y float32 (B,H,P), new state)."""
    x, xp = _req(x)
    Bsz, H, P = x.shape
    state = np.array(state, order="C", copy=True)
    N = state.shape[-1]
    assert state.shape == (Bsz, H, P, N)
    B, bp = _req(B)
    C_, cp = _req(C_)
    G = B.shape[1]
    dt, dp = _req(np.broadcast_to(np.asarray(dt, np.int8), (Bsz, H, P)))
    A_log, ap = _req(np.broadcast_to(np.asarray(A_log, np.int8), (H, P, N)))
    f32 = lambda a: np.ascontiguousarray(np.asarray(a, np.float32).reshape(-1))
    vp = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
    Dd = None if D is None else np.ascontiguousarray(np.broadcast_to(np.asarray(D, np.int8), (H, P)))
    db = None if dt_bias is None else np.ascontiguousarray(np.broadcast_to(np.asarray(dt_bias, np.float32), (H, P)))
    grouped = head_range is not None
    xs, sB, sC, ss = f32(x_scale), f32(s_B), f32(s_C), f32(state_scale)
    hr = None if not grouped else np.ascontiguousarray(head_range, np.int32)
    dr = None if not grouped else np.ascontiguousarray(dim_range, np.int32)
    nhg, ndg = (hr.shape[1], dr.shape[2]) if grouped else (0, 0)
    if grouped:
        assert xs.size == G * nhg * ndg and sB.size == G and sC.size == G and ss.size == G * nhg * ndg * N
    else:
        assert xs.size == 1 and sB.size == 1 and sC.size == 1 and ss.size == 1
    y = np.empty((Bsz, H, P), np.float32)
    if state.dtype == np.float32:
        s8, s32 = None, vp(state)
    else:
        assert state.dtype == np.int8
        s8, s32 = vp(state), None
    lib().qo_ssm_update_heads(s8, s32, xp, dp, ap, bp, cp, vp(Dd), vp(db), _opt(z), vp(xs), vp(ss), vp(sB), vp(sC),
                              vp(hr), vp(dr), _f(s_dt), _f(s_A), _f(s_D), _f(s_z), Bsz, H, P, N, G, nhg, ndg,
                              int(softplus), vp(y))
    return y, state


def gemm_w8a8(a, w, s_a, s_b, round_half_away=False):
    """a int8 (M,K), w int8 (N,K), s_a fp32 (1|M), s_b fp32 (1|N).
    Returns (acc int32 (M,N), fp32 value before the cast, int8 cast)."""
    a, ap = _req(a)
    w, wp = _req(w)
    s_a = np.ascontiguousarray(np.asarray(s_a, np.float32).reshape(-1))
    s_b = np.ascontiguousarray(np.asarray(s_b, np.float32).reshape(-1))
    M, K = a.shape
    N = w.shape[0]
    acc = np.empty((M, N), np.int32)
    f = np.empty((M, N), np.float32)
    q = np.empty((M, N), np.int8)
    lib().qo_gemm_w8a8(ap, wp, s_a.ctypes.data_as(C.c_void_p), s_a.size, s_b.ctypes.data_as(C.c_void_p), s_b.size,
                       M, N, K, int(round_half_away), acc.ctypes.data_as(C.c_void_p),
                       f.ctypes.data_as(C.c_void_p), q.ctypes.data_as(C.c_void_p))
    return acc, f, q


def gemm_w4a8(a, codes, s_group, s_channel, s_token, group_size=128):
    """a int8 (M,K); codes uint8 (N,K) 4-bit codes; s_group fp16 (K/128,N) or None (per-channel);
    s_channel fp32 (N); s_token fp32 (1|M).
    Returns (w8 int8 (N,K) expanded weights, acc int32 (M,N), fp32 value before the cast, int8 cast)."""
    a, ap = _req(a)
    codes, cp = _req(codes, np.uint8)
    M, K = a.shape
    N = codes.shape[0]
    if s_group is not None:
        sg = np.ascontiguousarray(np.asarray(s_group, np.float16).astype(np.float32).reshape(-1, N))
        sgp = sg.ctypes.data_as(C.c_void_p)
    else:
        sgp, group_size = None, -1
    sc = np.ascontiguousarray(np.asarray(s_channel, np.float32).reshape(-1))
    st = np.ascontiguousarray(np.asarray(s_token, np.float32).reshape(-1))
    w8 = np.empty((N, K), np.int8)
    acc = np.empty((M, N), np.int32)
    f = np.empty((M, N), np.float32)
    q = np.empty((M, N), np.int8)
    lib().qo_gemm_w4a8(ap, cp, sgp, sc.ctypes.data_as(C.c_void_p), st.ctypes.data_as(C.c_void_p), st.size,
                       M, N, K, group_size, w8.ctypes.data_as(C.c_void_p), acc.ctypes.data_as(C.c_void_p),
                       f.ctypes.data_as(C.c_void_p), q.ctypes.data_as(C.c_void_p))
    return w8, acc, f, q


class _QoSsdDims(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("batch", "seqlen", "nheads", "headdim", "dstate", "ngroups", "chunk",
                                       "softplus", "dt_is_f32", "D_has_hdim", "nhead_groups", "ndim_groups")] + \
               [("dt_min", C.c_float), ("dt_max", C.c_float)]


def ssd_fwd(x, dt, A_log, B, C_, D=None, z=None, dt_bias=None, *, chunk_size, x_scale, s_dt=1.0, s_A, s_B, s_C,
            s_D=0.0, s_z=0.0, state_scale=None, head_range=None, dim_range=None, softplus=True,
            dt_limit=(0.0, float("inf")), stages=False):
    """x int8 (B,L,H,P); dt int8 or float32 (B,L,H) (float32 = already processed); A_log int8 (H);
    B, C int8 (B,L,G,N); D int8 (H) or (H,P); z int8 like x; dt_bias float (H) holding fp16 values.
    x_scale / s_B / s_C / state_scale: scalars, or grouped arrays with head_range (G,hg) and
    dim_range (G,hg,dg) int32 cumulative end indices.
    Returns dict(y float32 (B,L,H,P) before the fp16 cast, final_f32, final_i8 [, dt, dA_cumsum, CB,
    chunk_states, prev_states with stages=True])."""
    x, xp = _req(x)
    Bsz, L, H, P = x.shape
    B, bp = _req(B)
    C_, cp = _req(C_)
    G, N = B.shape[2], B.shape[3]
    A_log, ap = _req(A_log)
    dt = np.ascontiguousarray(dt)
    dt_is_f32 = dt.dtype == np.float32
    assert dt_is_f32 or dt.dtype == np.int8
    grouped = head_range is not None
    dims = _QoSsdDims(Bsz, L, H, P, N, G, chunk_size, int(softplus), int(dt_is_f32),
                      int(D is not None and np.asarray(D).ndim == 2),
                      head_range.shape[1] if grouped else 0, dim_range.shape[2] if grouped else 0,
                      float(dt_limit[0]), float(min(dt_limit[1], 3.0e38)))
    f32 = lambda a: np.ascontiguousarray(np.asarray(a, np.float32).reshape(-1))
    xs, sB, sC = f32(x_scale), f32(s_B), f32(s_C)
    ss = f32(state_scale if state_scale is not None else 1.0)
    dbias = None if dt_bias is None else f32(np.asarray(dt_bias, np.float16))
    hr = None if not grouped else np.ascontiguousarray(head_range, np.int32)
    dr = None if not grouped else np.ascontiguousarray(dim_range, np.int32)
    nc = (L + chunk_size - 1) // chunk_size
    out = dict(y=np.zeros((Bsz, L, H, P), np.float32), final_f32=np.empty((Bsz, H, P, N), np.float32),
               final_i8=np.empty((Bsz, H, P, N), np.int8))
    if stages:
        out.update(dt=np.empty((Bsz, H, nc, chunk_size), np.float32), dA_cumsum=np.empty((Bsz, H, nc, chunk_size), np.float32),
                   CB=np.zeros((Bsz, nc, G, chunk_size, chunk_size), np.float32),
                   chunk_states=np.empty((Bsz, nc, H, P, N), np.float32), prev_states=np.empty((Bsz, nc, H, P, N), np.float32))
    vp = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
    lib().qo_ssd_fwd(C.byref(dims), xp, vp(dt), ap, bp, cp, _opt(D), _opt(z), vp(dbias), vp(xs), vp(hr), vp(dr),
                     _f(s_dt), _f(s_A), vp(sB), vp(sC), _f(s_D), _f(s_z), vp(ss),
                     vp(out["y"]), vp(out["final_f32"]), vp(out["final_i8"]),
                     vp(out.get("dt")), vp(out.get("dA_cumsum")), vp(out.get("CB")), vp(out.get("chunk_states")),
                     vp(out.get("prev_states")))
    return out


def _legendre(a, q):
    a %= q
    if a == 0:
        return 0
    return 1 if any((x * x) % q == a for x in range(1, q)) else -1


def hadamard_special(S):
    """The fixed S x S Hadamard matrix (+1/-1, int8) of the reference's 12N / 40N transforms
    (csrc/hadamard/code_gen.py: ``had_12_paley``, ``had_40_tpal``), built from the definitions:
    12: Paley's second construction for q = 5; 40: [[P, P], [P, -P]] with P the 20 x 20 Paley matrix for
    q = 19 (first row + - ... -, first column +, core delta - chi(k - i))."""
    if S == 12:
        C6 = np.zeros((6, 6), int)
        C6[0, 1:] = 1
        C6[1:, 0] = 1
        for i in range(1, 6):
            for k in range(1, 6):
                C6[i, k] = _legendre(k - i, 5)
        blk = {0: [[1, -1], [-1, -1]], 1: [[1, 1], [1, -1]], -1: [[-1, -1], [-1, 1]]}
        H = np.zeros((12, 12), int)
        for i in range(6):
            for k in range(6):
                H[2 * i:2 * i + 2, 2 * k:2 * k + 2] = blk[int(C6[i, k])]
        return H.astype(np.int8)
    if S == 40:
        P = np.ones((20, 20), int)
        P[0, 1:] = -1
        for i in range(1, 20):
            for k in range(1, 20):
                P[i, k] = 1 if i == k else -_legendre(k - i, 19)
        return np.block([[P, P], [P, -P]]).astype(np.int8)
    raise ValueError("S must be 12 or 40")


def hadamard_split(dim):
    """(S, M) with dim == S * M, the way quamba/hadamard_utils.py:33-47 picks the transform."""
    S = 12 if dim % 12 == 0 else (40 if dim % 40 == 0 else 1)
    M = dim // S
    assert M & (M - 1) == 0 and M > 0, "dim must be S * 2^k"
    return S, M


def hadamard_quant(x, scale):
    """x float16/float32 (..., dim) -> int8 of round(H x * scale)."""
    x = np.asarray(x)
    dim = x.shape[-1]
    S, _ = hadamard_split(dim)
    x2 = np.ascontiguousarray(x.reshape(-1, dim).astype(np.float32))
    out = np.empty(x2.shape, np.int8)
    signs = hadamard_special(S) if S > 1 else np.ones((1, 1), np.int8)
    signs = np.ascontiguousarray(signs)
    fp = lambda a: a.ctypes.data_as(C.c_void_p)
    lib().qo_hadamard_quant(fp(x2), fp(out), x2.shape[0], dim, S, fp(signs), _f(scale))
    return out.reshape(x.shape)


def rmsnorm_gated(x, weight, qz=None, *, eps, z_scale=0.0, group_size=None, norm_before_gate=True, out_mode="f16",
                  out_scale=None):
    """Gated RMS norm of quamba/triton/quant_normgated.py:34-82, evaluated in float64 (the kernel's fp32
    tree sums have no fixed order, so this restatement keeps the formula exact and leaves the last bit of
    the row statistic to the tolerance of the comparison).
    x float16 (M, N); weight float16 (N); qz int8 (M, N) or None.  Returns (y float64 (M, N) before the
    output cast, q, scales): q is float16 (out_mode "f16"), int8 with ``out_scale`` ("static") or int8 with
    the per-(row, group) scale max(y)/127 ("dynamic", scales float32 (groups, M))."""
    x = np.asarray(x, np.float16).astype(np.float64)
    M, N = x.shape
    g = N if group_size is None else group_size
    w = np.asarray(weight, np.float16).astype(np.float64)
    gate = None
    if qz is not None:
        z = np.float64(np.float32(z_scale)) * np.asarray(qz, np.int8).astype(np.float64)
        gate = z / (1.0 + np.exp(-z))
        if not norm_before_gate:
            x = x * gate                                                       # :48-50
    xg = x.reshape(M, N // g, g)
    var = (xg * xg).sum(axis=2, keepdims=True) / g                             # :55-56
    rstd = 1.0 / np.sqrt(var + np.float64(np.float32(eps)))                    # :58
    y = (xg * rstd).reshape(M, N) * w[None, :]                                 # :65-66
    if gate is not None and norm_before_gate:
        y = y * gate                                                           # :67-69
    if out_mode == "f16":
        return y, y.astype(np.float16), None
    if out_mode == "static":
        s = np.float64(np.float32(out_scale))
        return y, np.clip(np.rint(y / s), -128, 127).astype(np.int8), None     # :74-75
    s = y.reshape(M, N // g, g).max(axis=2) / 127.0                            # :77 (max, not max |.|)
    q = np.clip(np.rint(y.reshape(M, N // g, g) / s[:, :, None]), -128, 127).astype(np.int8).reshape(M, N)
    return y, q, np.ascontiguousarray(s.T).astype(np.float32)                  # scale index = group * M + row

"""GPU parity of the Mamba2 SSD chunk scan and its single-step update against the CPU oracle.
fp16 outputs: rtol 1e-2 / atol 1e-2 on the values themselves, every output; fp32 states 1e-3 relative; int8 states at most
one step off, and only where the un-rounded quotient lies within 2e-3 of a rounding tie."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import Quamba2ChunkScan, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _oracle(d, chunk, **kw):
    return oracle.ssd_fwd(d["x"], kw.pop("dt", d["dt"]), d["A_log"], d["B"], d["C"], d["D"], d["z"], d["dt_bias"],
                          chunk_size=chunk, x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                          s_D=d["s_D"], s_z=d["s_z"], head_range=d["head_range"], dim_range=d["dim_range"], **kw)


def _gpu(d, dev, chunk, state_scale=None, dt=None, final_dtype=torch.float32, **kw):
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    return ops.ssd_chunk_scan_combined_fwd(
        _t(d["x"], dev), s(d["x_scale"]), _t(d["dt"] if dt is None else dt, dev), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
        _t(d["B"], dev), s(d["s_B"]), _t(d["C"], dev), s(d["s_C"]), None if state_scale is None else s(state_scale), chunk,
        q_D=_t(d["D"], dev), D_scale=s(d["s_D"]), q_z=_t(d["z"], dev), z_scale=s(d["s_z"]), dt_bias=_t(d["dt_bias"], dev),
        dt_softplus=True, x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev),
        final_state_dtype=final_dtype, **kw)


def _check_y(y_gpu, y_ref):
    """The bar of the fp16 scan outputs, on the values themselves: |got - want| <= 1e-2 + 1e-2 |want| for every output.
    Measured on MI355X over the cases of this file (synthetic activations with outlier channels): no output beyond the
    bar, the farthest at 0.9 of it."""
    got = y_gpu.float().cpu().numpy()
    want = y_ref.astype(np.float16).astype(np.float32)
    bar = 1e-2 + 1e-2 * np.abs(want)
    err = np.abs(got - want)
    assert (err <= bar).all(), f"{int((err > bar).sum())} of {err.size} outputs beyond rtol 1e-2 / atol 1e-2, largest error / bar = {(err / bar).max():.2f}"
    assert np.sum((got - y_ref) ** 2) / np.sum(y_ref ** 2) < 1e-6


# batch, seqlen, nheads, dstate, ngroups, chunk
SHAPES = [(1, 64, 2, 128, 1, 64), (2, 33, 4, 128, 1, 64), (1, 89, 4, 64, 2, 64), (2, 300, 8, 64, 2, 128),
          (1, 512, 8, 128, 1, 256), (1, 1024, 4, 128, 1, 256), (1, 130, 4, 128, 4, 128),
          # chunks of 256 with a ragged last chunk: 128 states (entering state and upper B rows share LDS) and 64
          (1, 600, 4, 128, 2, 256), (2, 700, 4, 64, 1, 256),
          # fewer states than the kernels are built for (the 16-state row of test_ssd_combined.py:25, and 32, 96)
          (1, 33, 24, 16, 1, 128), (2, 200, 4, 32, 2, 64), (1, 150, 4, 96, 1, 128)]


@pytest.mark.parametrize("B,L,H,N,G,Q", SHAPES)
def test_forward_matches_oracle(dev, B, L, H, N, G, Q):
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=L + H)
    ref = _oracle(d, Q)
    y, final = _gpu(d, dev, Q)
    assert y.shape == (B, L, H, 64) and y.dtype == torch.float16 and final.shape == (B, H, 64, N)
    _check_y(y, ref["y"])
    got = final.cpu().numpy()
    assert np.abs(got - ref["final_f32"]).max() <= 1e-3 * np.abs(ref["final_f32"]).max()


# Heads of 128, 192 and 256 channels run on the matrix-core kernels as two, three and four heads of 64 that share the
# head's step sizes, decay and skip weight.  Shapes outside what those kernels are built for (head dimensions that are
# not multiples of 64, state counts other than 64 and 128, chunks other than 64, 128 or 256 steps) run on the
# library's general kernels, to the same bars.
# batch, seqlen, nheads, headdim, dstate, ngroups, chunk
GENERAL_SHAPES = [(1, 100, 4, 128, 128, 1, 64),      # the head dimension of the larger Mamba2 variants
                  (2, 300, 2, 256, 64, 2, 128),
                  (1, 520, 3, 192, 128, 1, 256),
                  (1, 100, 4, 128, 128, 1, 96),      # the same head dimension on the general kernels
                  (2, 77, 4, 32, 16, 2, 32),         # small everything
                  (1, 300, 2, 64, 256, 1, 128),      # more states than one tile pair
                  (1, 200, 4, 64, 128, 1, 512),      # one chunk longer than the sequence
                  (1, 700, 2, 64, 64, 2, 512),       # a whole and a ragged chunk of 512
                  (2, 150, 4, 96, 48, 2, 100),       # nothing a multiple of 64
                  (1, 130, 6, 40, 24, 3, 48),
                  (1, 65, 2, 256, 16, 1, 60),        # the largest head dimension
                  (1, 33, 3, 1, 1, 1, 7)]            # the smallest


@pytest.mark.parametrize("B,L,H,P,N,G,Q", GENERAL_SHAPES)
def test_forward_of_other_shapes_matches_oracle(dev, B, L, H, P, N, G, Q):
    d = synth.mamba2_ssd_inputs(B, L, H, P, N, G, seed=L + P)
    ref = _oracle(d, Q)
    y, final = _gpu(d, dev, Q)
    assert y.shape == (B, L, H, P) and y.dtype == torch.float16 and final.shape == (B, H, P, N)
    _check_y(y, ref["y"])
    got = final.cpu().numpy()
    assert np.abs(got - ref["final_f32"]).max() <= 1e-3 * np.abs(ref["final_f32"]).max()


# (96 channels, 80 states, chunks of 96: the general kernels; 128 channels in dim groups of 32, i.e. two to each half of
# a head, and 192 channels in dim groups of 48 that straddle the thirds: the matrix-core kernels)
@pytest.mark.parametrize("P,N,Q,ndg", [(96, 80, 96, 3), (128, 128, 128, 4), (192, 64, 64, 4)])
@pytest.mark.parametrize("with_z,d_has_hdim", [(True, False), (False, True)])
def test_other_shapes_with_grouped_scales_z_gate_and_int8_state(dev, with_z, d_has_hdim, P, N, Q, ndg):
    B, L, H, G = 2, 150, 8, 2
    d = synth.mamba2_ssd_inputs(B, L, H, P, N, G, seed=6, grouped=True, nhead_groups=2, ndim_groups=ndg, with_z=with_z)
    if d_has_hdim:
        d["D"] = np.random.default_rng(1).integers(60, 128, (H, P)).astype(np.int8)
    ref = _oracle(d, Q)
    g = np.random.default_rng(2)
    state_scale = (np.abs(ref["final_f32"]).max() / 127 * g.uniform(0.8, 1.2, (G, 2, ndg, N))).astype(np.float32)
    ref = _oracle(d, Q, state_scale=state_scale)
    y, final = _gpu(d, dev, Q, state_scale=state_scale, final_dtype=torch.int8)
    _check_y(y, ref["y"])
    diff = np.abs(final.cpu().numpy().astype(int) - ref["final_i8"].astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02
    assert np.abs(ref["final_i8"]).max() > 100


def test_unaligned_tensors_take_the_general_kernels_with_the_same_result(dev):
    """The matrix-core kernels read x, B, C and write the output in aligned 16-byte pieces; views that start elsewhere
    run on the general kernels: same bars against the oracle, and close to the aligned call's own output."""
    B, L, H, N, G, Q = 1, 200, 4, 128, 1, 128
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=21)
    ref = _oracle(d, Q)
    y0, f0 = _gpu(d, dev, Q)

    def shifted(a):
        flat = torch.empty(a.size + 1, dtype=torch.int8, device=dev)
        flat[1:] = torch.from_numpy(np.ascontiguousarray(a)).to(dev).reshape(-1)
        v = flat[1:].view(a.shape)
        assert v.data_ptr() % 16 == 1 and v.is_contiguous()
        return v

    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    y1, f1 = ops.ssd_chunk_scan_combined_fwd(
        shifted(d["x"]), s(d["x_scale"]), _t(d["dt"], dev), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
        shifted(d["B"]), s(d["s_B"]), shifted(d["C"]), s(d["s_C"]), None, Q, q_D=_t(d["D"], dev), D_scale=s(d["s_D"]),
        dt_bias=_t(d["dt_bias"], dev), dt_softplus=True, final_state_dtype=torch.float32)
    _check_y(y1, ref["y"])
    np.testing.assert_allclose(f1.cpu().numpy(), f0.cpu().numpy(), rtol=1e-4, atol=1e-5 * np.abs(ref["final_f32"]).max())
    assert (y1.float() - y0.float()).abs().max() <= 2e-2 * y0.float().abs().max()


def test_preparation_stages_match_the_oracle(dev):
    # what the preparation kernel leaves in the workspace: step sizes and their running sums (C B^T is formed inside
    # the chunk scan and never stored; the outputs below depend on every element of it at or below the diagonal)
    B, L, H, N, G, Q = 2, 200, 4, 128, 2, 64
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=77)
    ref = _oracle(d, Q, stages=True)
    y, final, ws = _gpu(d, dev, Q, return_workspace=True)
    nc = (L + Q - 1) // Q
    a256 = lambda v: (v + 255) & ~255
    off, parts = 0, {}
    for name, shape in [("dt", (B, H, nc, Q)), ("dA_cumsum", (B, H, nc, Q))]:
        n = int(np.prod(shape)) * 4
        parts[name] = ws[off:off + n].view(torch.float32).view(shape).cpu().numpy()
        off = a256(off + n)
    np.testing.assert_allclose(parts["dt"], ref["dt"], rtol=1e-5, atol=1e-9)
    np.testing.assert_allclose(parts["dA_cumsum"], ref["dA_cumsum"], rtol=1e-5, atol=1e-8)
    _check_y(y, ref["y"])


# 16, 32 and 96 states run as 64 or 128 with zero B and C columns added; the grouped state scale then has fewer
# columns than the kernel walks (the wrapper pads it), which is what these cases pin
@pytest.mark.parametrize("N", [128, 16, 32, 96])
@pytest.mark.parametrize("with_z,d_has_hdim", [(True, False), (False, True)])
def test_grouped_scales_z_gate_and_int8_state(dev, with_z, d_has_hdim, N):
    B, L, H, G, Q = 2, 150, 16, 2, 128
    d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=5, grouped=True, nhead_groups=4, ndim_groups=4, with_z=with_z)
    if d_has_hdim:
        d["D"] = np.random.default_rng(1).integers(60, 128, (H, 64)).astype(np.int8)
    ref = _oracle(d, Q)
    g = np.random.default_rng(2)
    state_scale = (np.abs(ref["final_f32"]).max() / 127 * g.uniform(0.8, 1.2, (G, 4, 4, N))).astype(np.float32)
    ref = _oracle(d, Q, state_scale=state_scale)
    y, final = _gpu(d, dev, Q, state_scale=state_scale, final_dtype=torch.int8)
    _check_y(y, ref["y"])
    assert final.dtype == torch.int8
    diff = np.abs(final.cpu().numpy().astype(int) - ref["final_i8"].astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02
    assert np.abs(ref["final_i8"]).max() > 100


def test_fp32_step_sizes_entry_point(dev):
    d = synth.mamba2_ssd_inputs(1, 256, 4, 64, 128, 1, seed=9)
    dt_proc = synth.softplus(d["dt"].astype(np.float32) * d["s_dt"] + d["dt_bias"].astype(np.float32)[None, None]).astype(np.float32)
    ref = _oracle(d, 128, dt=dt_proc)
    y, final = _gpu(d, dev, 128, dt=dt_proc)
    _check_y(y, ref["y"])


def test_module_forward_then_update_continue_the_sequence(dev):
    B, L, H, N, G, Q = 2, 128, 8, 128, 2, 64
    d = synth.mamba2_ssd_inputs(B, L + 3, H, 64, N, G, seed=13, grouped=True, nhead_groups=2, ndim_groups=2)
    ref = _oracle(d, 131)                     # one chunk covering everything: the recurrence itself
    ref = _oracle(d, Q)
    A_log = torch.from_numpy(d["A_log"].astype(np.float32) * d["s_A"]).to(dev)
    q = Quamba2ChunkScan.from_fp16(
        H * 64, 64, N, G, torch.from_numpy(d["x_scale"]), _t(d["head_range"], dev), _t(d["dim_range"], dev), A_log, Q,
        ssm_state_scale=torch.ones(G, 2, 2, N), D=torch.ones(H, device=dev), dt_bias=_t(d["dt_bias"], dev),
        dt_scale=torch.tensor(float(d["s_dt"])), B_scale=torch.from_numpy(d["s_B"]), C_scale=torch.from_numpy(d["s_C"]))
    np.testing.assert_array_equal(q.A_log.cpu().numpy(), d["A_log"])
    assert q.dt_bias.dtype == torch.float16 and q.x_scales.shape == (G, 2, 2) and q.ssm_state_scale.shape == (G, 2, 2, N)
    cut = lambda a: _t(a[:, :L], dev)
    y, state = q(cut(d["x"]), cut(d["dt"]), cut(d["B"]), cut(d["C"]), return_final_states=True, state_dtype=torch.float32)
    _check_y(y, ref["y"][:, :L])
    # the steps after the prefill: against the oracle's single step from the oracle's own state after L steps (the bar
    # of the fp16 outputs), and against the chunked form run over L + 3 steps, which is the same mathematics with
    # other roundings (fp16 states and weights there, an fp32 state here): a looser, absolute bar
    head = dict(d, **{k: d[k][:, :L] for k in ("x", "dt", "B", "C")})
    st_ref = _oracle(head, Q)["final_f32"]
    assert np.abs(state.cpu().numpy() - st_ref).max() <= 2e-3 * np.abs(st_ref).max()
    for t in range(L, L + 3):
        yt = q.update(state, _t(d["x"][:, t].reshape(B, -1), dev), _t(d["dt"][:, t], dev), _t(d["B"][:, t].reshape(B, -1), dev),
                      _t(d["C"][:, t].reshape(B, -1), dev))
        y_ref, st_ref = oracle.ssm_update_heads(
            st_ref, d["x"][:, t], d["dt"][:, t, :, None], d["A_log"][:, None, None], d["B"][:, t], d["C"][:, t], d["D"][:, None],
            d["dt_bias"].astype(np.float32)[:, None], None, x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"],
            s_C=d["s_C"], s_D=d["s_D"], state_scale=np.ones((G, 2, 2, N), np.float32), head_range=d["head_range"], dim_range=d["dim_range"])
        got = yt.float().cpu().numpy().reshape(B, H, 64)
        np.testing.assert_allclose(got, y_ref.astype(np.float16).astype(np.float32), rtol=1e-2, atol=1e-2)
        np.testing.assert_allclose(got, ref["y"][:, t].astype(np.float16).astype(np.float32), rtol=1e-2, atol=3e-2)
    assert np.abs(state.cpu().numpy() - st_ref).max() <= 2e-3 * np.abs(st_ref).max()


def _update_step_inputs(B, H, N, G, steps, seed):
    d = synth.mamba2_ssd_inputs(B, steps, H, 64, N, G, seed=seed, grouped=True, nhead_groups=4, ndim_groups=4, with_z=True)
    g = np.random.default_rng(seed)
    d["state_scale"] = (0.004 * g.uniform(0.5, 1.5, (G, 4, 4, N))).astype(np.float32)
    d["state0"] = g.integers(-127, 128, (B, H, 64, N)).astype(np.int8)
    return d


def _oracle_step(d, t, state):
    return oracle.ssm_update_heads(state, d["x"][:, t], d["dt"][:, t, :, None], d["A_log"][:, None, None], d["B"][:, t],
                                   d["C"][:, t], d["D"][:, None], d["dt_bias"].astype(np.float32)[:, None], d["z"][:, t],
                                   x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                                   s_D=d["s_D"], s_z=d["s_z"], state_scale=d["state_scale"], head_range=d["head_range"],
                                   dim_range=d["dim_range"])


def _expand_state_scale(d, H, G):
    """state scale per (head, p, n) from the group tables, for the tie test below"""
    hpg, hs, ds = H // G, (H // G) // 4, 64 // 4
    h = np.arange(H)
    return d["state_scale"][h[:, None] // hpg, (h[:, None] % hpg) // hs, np.arange(64)[None, :] // ds]      # (H, 64, N)


def _check_int8_state(got, want_i8, h_f32, scale_hpn):
    """at most one step off, and only where the quotient the rounding sees is within 2e-3 of a tie (the kernel's exp is
    the hardware's, the oracle's is libm's)"""
    diff = np.abs(got.astype(int) - want_i8.astype(int))
    assert diff.max() <= 1
    q = h_f32.astype(np.float64) / scale_hpn[None].astype(np.float64)
    near_tie = np.abs(np.abs(q - np.floor(q)) - 0.5) < 2e-3
    assert not (diff != 0)[~near_tie].any()
    assert (diff != 0).mean() < 0.01


# the three rows of the reference's test_qchunkscan_group_heads_update (quamba/tests/test_ssd_combined.py:40-44)
@pytest.mark.parametrize("B,H,N,G", [(1, 24, 16, 1), (4, 80, 128, 1), (4, 128, 128, 8)])
def test_grouped_int8_state_update_matches_oracle(dev, B, H, N, G):
    steps = 6
    d = _update_step_inputs(B, H, N, G, steps, seed=H + N)
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    nheads = H
    state = _t(d["state0"], dev)
    ref_state = d["state0"]
    scale_hpn = _expand_state_scale(d, H, G)
    A3 = _t(d["A_log"], dev).view(nheads, 1, 1).expand(nheads, 64, N)
    D2 = _t(d["D"], dev).view(nheads, 1).expand(nheads, 64)
    b2 = _t(d["dt_bias"], dev).view(nheads, 1).expand(nheads, 64)
    saw_big = False
    for t in range(steps):
        deq = (ref_state.astype(np.float32) * scale_hpn[None]).astype(np.float32)
        _, h_f32 = _oracle_step(d, t, deq)                     # the fp32 state the requantisation rounds
        y_ref, ref_state = _oracle_step(d, t, ref_state)
        dt3 = _t(d["dt"][:, t], dev).unsqueeze(-1).expand(B, nheads, 64)
        y = ops.sscan_update(state, _t(d["x"][:, t], dev), s(d["x_scale"]), dt3, s(d["s_dt"]), A3, s(d["s_A"]),
                             s(d["state_scale"]), _t(d["B"][:, t], dev), s(d["s_B"]), _t(d["C"][:, t], dev), s(d["s_C"]),
                             D2, s(d["s_D"]), _t(d["z"][:, t], dev), s(d["s_z"]), b2, None, True,
                             x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev))
        assert state.dtype == torch.int8 and y.dtype == torch.float16
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref.astype(np.float16).astype(np.float32), rtol=1e-2, atol=1e-2)
        _check_int8_state(state.cpu().numpy(), ref_state, h_f32, scale_hpn)
        saw_big = saw_big or np.abs(ref_state).max() > 100
        state.copy_(_t(ref_state, dev))                        # both sides take the next step from the same state
    assert saw_big


def test_grouped_int8_state_update_strided_state_and_odd_state_count(dev):
    # dstate % 4 != 0 and a state tensor that is a slice of a wider one: the element-wise kernel
    B, H, N, G, steps = 3, 8, 30, 2, 5
    d = _update_step_inputs(B, H, N, G, steps, seed=41)
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    wide = torch.zeros((B, H, 64, N + 3), dtype=torch.int8, device=dev)
    state = wide[..., 1:N + 1]
    state.copy_(_t(d["state0"], dev))
    ref_state = d["state0"]
    scale_hpn = _expand_state_scale(d, H, G)
    A3 = _t(d["A_log"], dev).view(H, 1, 1).expand(H, 64, N)
    b2 = _t(d["dt_bias"], dev).view(H, 1).expand(H, 64)
    d["D"] = None
    for t in range(steps):
        deq = (ref_state.astype(np.float32) * scale_hpn[None]).astype(np.float32)
        _, h_f32 = _oracle_step_noD(d, t, deq)
        y_ref, ref_state = _oracle_step_noD(d, t, ref_state)
        dt3 = _t(d["dt"][:, t], dev).unsqueeze(-1).expand(B, H, 64)
        y = ops.sscan_update(state, _t(d["x"][:, t], dev), s(d["x_scale"]), dt3, s(d["s_dt"]), A3, s(d["s_A"]),
                             s(d["state_scale"]), _t(d["B"][:, t], dev), s(d["s_B"]), _t(d["C"][:, t], dev), s(d["s_C"]),
                             None, None, _t(d["z"][:, t], dev), s(d["s_z"]), b2, None, True,
                             x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev))
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref.astype(np.float16).astype(np.float32), rtol=1e-2, atol=1e-2)
        _check_int8_state(state.cpu().numpy(), ref_state, h_f32, scale_hpn)
        state.copy_(_t(ref_state, dev))
    assert (wide[..., 0] == 0).all() and (wide[..., N + 1:] == 0).all()        # nothing written outside the view


def _oracle_step_noD(d, t, state):
    return oracle.ssm_update_heads(state, d["x"][:, t], d["dt"][:, t, :, None], d["A_log"][:, None, None], d["B"][:, t],
                                   d["C"][:, t], None, d["dt_bias"].astype(np.float32)[:, None], d["z"][:, t],
                                   x_scale=d["x_scale"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                                   s_z=d["s_z"], state_scale=d["state_scale"], head_range=d["head_range"],
                                   dim_range=d["dim_range"])


def test_errors(dev):
    d = synth.mamba2_ssd_inputs(1, 64, 2, 64, 128, 1, seed=1)
    with pytest.raises(NotImplementedError):
        _gpu(d, dev, 2048)                                # chunks of more than 1024 steps
    with pytest.raises(NotImplementedError, match="seq_idx"):
        _gpu(d, dev, 64, seq_idx=torch.zeros(1, 64, device=dev))
    d2 = synth.mamba2_ssd_inputs(1, 8, 1, 320, 16, 1, seed=1)
    with pytest.raises(NotImplementedError):
        _gpu(d2, dev, 64)                                 # head dimensions above 256

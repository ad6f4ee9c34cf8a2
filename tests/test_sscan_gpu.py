"""GPU parity of the Mamba1 selective scan (forward and single-step update) against the CPU oracle.
fp16 outputs: rtol 1e-2 / atol 1e-2; fp32 state: 1e-3 relative; int8 state: at most one step off."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import QSScan, ops, synth

pytestmark = pytest.mark.gpu

RTOL = ATOL = 1e-2
STATE_REL = 1e-3


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _s(v, dev):
    return torch.tensor([float(v)], dtype=torch.float32, device=dev)


def _oracle(d, s_state):
    return oracle.sscan_fwd(d["u"], d["dt"], d["A_log"], d["B"], d["C"], d["D"], d["dt_bias"], d["z"],
                            s_u=d["s_u"], s_delta=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                            s_D=d["s_D"], s_db=d["s_db"], s_z=d["s_z"], s_state=s_state)


def _gpu(d, dev, s_state, state_dtype):
    return ops.sscan_fwd(
        _t(d["u"], dev), _s(d["s_u"], dev), _t(d["dt"], dev), _s(d["s_dt"], dev), _t(d["A_log"], dev), _s(d["s_A"], dev),
        _t(d["B"][:, None], dev), _s(d["s_B"], dev), _t(d["C"][:, None], dev), _s(d["s_C"], dev), _s(s_state, dev),
        _t(d["D"], dev), _s(d["s_D"], dev), _t(d["z"], dev), _s(d["s_z"], dev) if d["z"] is not None else None,
        _t(d["dt_bias"], dev), _s(d["s_db"], dev), True, state_dtype=state_dtype)


def _check(y_gpu, y_ref):
    y16 = y_ref.astype(np.float16).astype(np.float32)
    got = y_gpu.float().cpu().numpy()
    np.testing.assert_allclose(got, y16, rtol=RTOL, atol=ATOL)
    r2 = np.sum((got - y_ref) ** 2) / max(np.sum(y_ref ** 2), 1e-30)
    assert r2 < 1e-5


# (batch, seqlen, dim, dstate): 130m/2.8b-shaped rows, ragged lengths, channel tails, wide states, and the
# 128-state rows of the reference's own list (test_qsscan.py:51-54: dims 5120 and 8192, here with fewer steps)
SHAPES = [(1, 512, 1536, 16), (2, 33, 1536, 16), (2, 89, 100, 16), (1, 1, 64, 16), (2, 2048 + 7, 96, 16),
          (2, 130, 72, 8), (1, 200, 40, 32), (1, 100, 24, 64), (1, 70, 8, 128), (1, 40, 6, 256),
          (4, 96, 5120, 128), (4, 40, 8192, 128),
          # wide states with many channels (four waves share a B/C tile): ragged channel tails, a padded state count
          (2, 70, 4170, 32), (2, 50, 2100, 64), (3, 33, 1400, 100),
          # aligned rows whose last tile is ragged (whole tiles by vector loads, the last one byte-wise), and one tile only
          (2, 48, 128, 16), (1, 80, 200, 16), (2, 16, 64, 16), (9, 176, 640, 16)]


@pytest.mark.parametrize("B,L,D,N", SHAPES)
def test_fwd_matches_oracle(dev, B, L, D, N):
    d = synth.mamba1_scan_inputs(B, L, D, N, seed=L + D)
    y_ref, st8_ref, st32_ref = _oracle(d, s_state=1.0)
    s_state = max(float(np.abs(st32_ref).max()), 1e-5) / 127.0
    _, st8_ref, _ = _oracle(d, s_state=s_state)
    y, x32 = _gpu(d, dev, s_state, torch.float32)
    assert y.shape == (B, L, D) and y.dtype == torch.float16 and x32.shape == (B, D, 1, N)
    _check(y, y_ref)
    got32 = x32[:, :, 0].cpu().numpy()
    assert np.abs(got32 - st32_ref).max() <= STATE_REL * np.abs(st32_ref).max()
    y2, x8 = _gpu(d, dev, s_state, torch.int8)
    assert torch.equal(y, y2)
    diff = np.abs(x8[:, :, 0].cpu().numpy().astype(int) - st8_ref.astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02


# (seqlen, dim, dstate, variant): a single sequence is scanned as 8, 8, 4 or 2 segments side by side, each segment
# a second time from the state its predecessors chain up to; with every lane mapping that can meet it
@pytest.mark.parametrize("L,D,N,variant", [(2048, 256, 16, None), (1536, 96, 16, "4x4"), (1024, 200, 16, "8x4"),
                                           (1024, 64, 16, "2x2"), (1056, 40, 32, None), (1024, 24, 64, None),
                                           (2048, 5120, 16, None),
                                           # wide states: four waves per workgroup (128 workgroups and more) and one
                                           (1024, 512, 128, None), (1024, 544, 64, None), (1024, 100, 100, None)])
def test_one_sequence_scanned_in_segments(dev, L, D, N, variant, monkeypatch):
    if variant:
        monkeypatch.setattr(ops, "SSCAN_MAPPING", ops.sscan_mapping(*map(int, variant.split("x"))))
    assert ops._sscan_segments(1, D, L) > 1
    d = synth.mamba1_scan_inputs(1, L, D, N, seed=L + D + 1)
    y_ref, _, st32_ref = _oracle(d, s_state=1.0)
    s_state = max(float(np.abs(st32_ref).max()), 1e-5) / 127.0
    _, st8_ref, _ = _oracle(d, s_state=s_state)
    y, x32 = _gpu(d, dev, s_state, torch.float32)
    assert y.shape == (1, L, D) and x32.shape == (1, D, 1, N)
    _check(y, y_ref)
    assert np.abs(x32[:, :, 0].cpu().numpy() - st32_ref).max() <= STATE_REL * np.abs(st32_ref).max()
    y8, x8 = _gpu(d, dev, s_state, torch.int8)
    assert torch.equal(y, y8) and x8.shape == (1, D, 1, N) and x8.dtype == torch.int8
    diff = np.abs(x8[:, :, 0].cpu().numpy().astype(int) - st8_ref.astype(int))
    assert diff.max() <= 1 and (diff != 0).mean() < 0.02
    # and against the same kernel walking the sequence in one piece
    monkeypatch.setattr(ops, "SSCAN_SEGMENT_MIN_STEPS", 0)
    y1, x1 = _gpu(d, dev, s_state, torch.float32)
    np.testing.assert_allclose(y.float().cpu().numpy(), y1.float().cpu().numpy(), rtol=2e-3, atol=2e-3)
    assert (x32 - x1).abs().max().item() <= 1e-4 * x1.abs().max().item()


# "<lanes per channel>x<waves>"; "8x4" is the eight-lane mapping, "0x<n>" the mixed launch (n workgroups of 64
# channels with four lanes per channel, the remaining channels with eight)
@pytest.mark.parametrize("variant", ["1x1", "2x1", "2x2", "4x1", "4x2", "4x4", "8x4", "0x1", "0x2"])
def test_every_lane_mapping_gives_the_same_answer(dev, variant, monkeypatch):
    monkeypatch.setattr(ops, "SSCAN_MAPPING", ops.sscan_mapping(*map(int, variant.split("x"))))
    d = synth.mamba1_scan_inputs(2, 300, 200, 16, seed=21)
    y_ref, _, st32_ref = _oracle(d, s_state=1.0)
    y, x32 = _gpu(d, dev, 1.0, torch.float32)
    _check(y, y_ref)
    assert np.abs(x32[:, :, 0].cpu().numpy() - st32_ref).max() <= STATE_REL * np.abs(st32_ref).max()


def test_fwd_without_z_d_and_bias(dev):
    d = synth.mamba1_scan_inputs(2, 77, 48, 16, seed=4, with_z=False)
    d["D"] = None
    d["dt_bias"] = None
    y_ref, _, _ = _oracle(d, 1.0)
    y, _ = _gpu(d, dev, 1.0, torch.float32)
    _check(y, y_ref)


def test_fwd_on_strided_mixer_views(dev):
    # x and z are the halves of in_proj's [2D][B][L] output viewed as (B, D, L); dt has its own buffer
    B, L, D, N = 2, 256, 128, 16
    d = synth.mamba1_scan_inputs(B, L, D, N, seed=8)
    buf = torch.zeros((2 * D, B, L), dtype=torch.int8, device=dev).transpose(0, 1)
    u, z = buf[:, :D], buf[:, D:]
    u.copy_(_t(d["u"], dev))
    z.copy_(_t(d["z"], dev))
    dt = torch.zeros((D, B, L), dtype=torch.int8, device=dev).transpose(0, 1)
    dt.copy_(_t(d["dt"], dev))
    y, _ = ops.sscan_fwd(u, _s(d["s_u"], dev), dt, _s(d["s_dt"], dev), _t(d["A_log"], dev), _s(d["s_A"], dev),
                         _t(d["B"][:, None], dev), _s(d["s_B"], dev), _t(d["C"][:, None], dev), _s(d["s_C"], dev),
                         _s(1.0, dev), _t(d["D"], dev), _s(d["s_D"], dev), z, _s(d["s_z"], dev),
                         _t(d["dt_bias"], dev), _s(d["s_db"], dev), True, state_dtype=torch.float32)
    _check(y, _oracle(d, 1.0)[0])


def test_fwd_unaligned_rows(dev):
    B, L, D, N = 2, 50, 20, 16               # row pitch 50: no 16-byte alignment anywhere
    d = synth.mamba1_scan_inputs(B, L, D, N, seed=12)
    y, _ = _gpu(d, dev, 1.0, torch.float32)
    _check(y, _oracle(d, 1.0)[0])


@pytest.mark.parametrize("B,D,N,fp32_state", [(1, 1536, 16, False), (64, 5120, 16, True), (3, 100, 16, False),
                                              (2, 192, 16, True), (3, 100, 16, True), (2, 64, 128, True), (2, 30, 8, False),
                                              (4, 5120, 128, False), (4, 8192, 128, True)])
def test_update_matches_oracle_over_several_steps(dev, B, D, N, fp32_state):
    steps = 5
    d = synth.mamba1_scan_inputs(B, steps, D, N, seed=D + N)
    g = np.random.default_rng(D)
    if fp32_state:
        st_ref = (0.1 * g.standard_normal((B, D, N))).astype(np.float32)
        s_state = 1.0
    else:
        st_ref = g.integers(-128, 128, (B, D, N)).astype(np.int8)
        s_state = 0.004
    st = _t(st_ref.copy(), dev)
    A, Dq, db = _t(d["A_log"], dev), _t(d["D"], dev), _t(d["dt_bias"], dev)
    for t in range(steps):
        y_ref, st_ref = oracle.sscan_update(st_ref, d["u"][:, :, t], d["dt"][:, :, t], d["A_log"], d["B"][:, :, t],
                                            d["C"][:, :, t], d["D"], d["dt_bias"], d["z"][:, :, t],
                                            s_x=d["s_u"], s_dt=d["s_dt"], s_A=d["s_A"], s_B=d["s_B"], s_C=d["s_C"],
                                            s_D=d["s_D"], s_db=d["s_db"], s_z=d["s_z"], s_state=s_state)
        y = ops.sscan_update(st, _t(d["u"][:, :, t], dev), _s(d["s_u"], dev), _t(d["dt"][:, :, t], dev),
                             _s(d["s_dt"], dev), A, _s(d["s_A"], dev), _s(s_state, dev), _t(d["B"][:, :, t], dev),
                             _s(d["s_B"], dev), _t(d["C"][:, :, t], dev), _s(d["s_C"], dev), Dq, _s(d["s_D"], dev),
                             _t(d["z"][:, :, t], dev), _s(d["s_z"], dev), db, _s(d["s_db"], dev), True)
        np.testing.assert_allclose(y.float().cpu().numpy(), y_ref.astype(np.float16).astype(np.float32),
                                   rtol=RTOL, atol=ATOL)
        got = st.cpu().numpy()
        if fp32_state:
            assert np.abs(got - st_ref).max() <= STATE_REL * np.abs(st_ref).max()
        else:
            diff = np.abs(got.astype(int) - st_ref.astype(int))
            assert diff.max() <= 1 and (diff != 0).mean() < 0.01
            st_ref = got.copy()              # follow the GPU's state so a one-step tie does not compound


@pytest.mark.parametrize("B,D,N,width,state_len,fp32_state", [(3, 100, 16, 4, 3, True), (64, 1536, 16, 4, 4, False),
                                                              (7, 300, 16, 4, 4, True), (3, 320, 16, 4, 4, True),
                                                              (2, 257, 8, 3, 2, True),
                                                              (5, 64, 16, 2, 2, False),
                                                              # a conv state of three codes per row, rows back to back: the
                                                              # fixed-shape kernel reads a row as one unaligned word
                                                              (64, 1536, 16, 4, 3, False), (7, 320, 16, 4, 3, True),
                                                              (1, 64, 16, 4, 3, True), (2, 100, 16, 4, 3, False)])
def test_decode_step_in_one_launch_equals_conv_update_then_state_update(dev, B, D, N, width, state_len, fp32_state):
    """qa_mamba1_decode_step against the two calls it stands for, bit for bit (conv output, conv state, y, state),
    over several steps; the two-call path is the one the oracle tests pin."""
    steps = 4
    g = torch.Generator(device=dev).manual_seed(B * D + width)
    ri = lambda *shape: torch.randint(-128, 128, shape, dtype=torch.int8, device=dev, generator=g)
    w, bias = ri(D, width), ri(D)
    A, Dq, db = ri(D, N), ri(D), ri(D)
    conv_a = ri(B, D, state_len)
    st_a = (torch.randn(B, D, N, device=dev, generator=g) * 0.1) if fp32_state else ri(B, D, N)
    conv_b, st_b = conv_a.clone(), st_a.clone()
    sc = [_s(v, dev) for v in (0.02, 0.02, 0.03, 0.03, 0.008, 0.04, 0.01, 0.004)]
    s_dt, s_A, s_B, s_C, s_D, s_z, s_db, s_state = sc
    for _ in range(steps):
        x, dt, z, Bv, Cv = ri(B, D), ri(B, D), ri(B, D), ri(B, N), ri(B, N)
        xc_a = ops.causal_conv1d_update(x, conv_a, 0.04, w, 0.004, 0.03, 0.004, bias, True)
        y_a = ops.sscan_update(st_a, xc_a, _s(0.03, dev), dt, s_dt, A, s_A, s_state, Bv, s_B, Cv, s_C, Dq, s_D, z, s_z, db, s_db, True)
        xc_b, y_b = ops.mamba1_decode_step(x, conv_b, 0.04, w, 0.004, 0.03, 0.004, bias, True, st_b, dt, s_dt, A, s_A, s_state,
                                           Bv, s_B, Cv, s_C, Dq, s_D, z, s_z, db, s_db, True)
        assert torch.equal(xc_a, xc_b) and torch.equal(conv_a, conv_b)
        assert torch.equal(y_a, y_b) and torch.equal(st_a, st_b)
    assert int(xc_a.abs().max()) > 10 and float(y_a.float().abs().max()) > 0.1


@pytest.mark.parametrize("state_len", [4, 3])
@pytest.mark.parametrize("fp32_state", [True, False])
def test_decode_step_without_optional_operands(dev, fp32_state, state_len):
    """The reference layer's layout (the kernel compiled for that shape; conv state of four codes per row, or three) with
    no skip weight, no gate, no dt bias, no conv bias and no SiLU: one launch against the two calls, bit for bit."""
    B, D, N = 5, 256, 16
    g = torch.Generator(device=dev).manual_seed(99)
    ri = lambda *shape: torch.randint(-128, 128, shape, dtype=torch.int8, device=dev, generator=g)
    w, A = ri(D, 4), ri(D, N)
    conv_a = ri(B, D, state_len)
    st_a = (torch.randn(B, D, N, device=dev, generator=g) * 0.1) if fp32_state else ri(B, D, N)
    conv_b, st_b = conv_a.clone(), st_a.clone()
    s_dt, s_A, s_B, s_C, s_state = (_s(v, dev) for v in (0.02, 0.02, 0.03, 0.03, 0.004))
    for _ in range(3):
        x, dt, Bv, Cv = ri(B, D), ri(B, D), ri(B, N), ri(B, N)
        xc_a = ops.causal_conv1d_update(x, conv_a, 0.04, w, 0.004, 0.03, 0.004, None, False)
        y_a = ops.sscan_update(st_a, xc_a, _s(0.03, dev), dt, s_dt, A, s_A, s_state, Bv, s_B, Cv, s_C)
        xc_b, y_b = ops.mamba1_decode_step(x, conv_b, 0.04, w, 0.004, 0.03, 0.004, None, False, st_b, dt, s_dt, A, s_A, s_state,
                                           Bv, s_B, Cv, s_C)
        assert torch.equal(xc_a, xc_b) and torch.equal(conv_a, conv_b)
        assert torch.equal(y_a, y_b) and torch.equal(st_a, st_b)
    assert float(y_a.float().abs().max()) > 0.01


def test_decode_step_in_one_launch_refuses_what_it_does_not_cover(dev):
    ri = lambda *shape: torch.randint(-128, 128, shape, dtype=torch.int8, device=dev)
    B, D, N = 2, 64, 32                                      # more than sixteen states
    with pytest.raises(NotImplementedError):
        ops.mamba1_decode_step(ri(B, D), ri(B, D, 3), 0.04, ri(D, 4), 0.004, 0.03, 0.004, None, True,
                               torch.zeros(B, D, N, device=dev), ri(B, D), _s(0.02, dev), ri(D, N), _s(0.02, dev), None,
                               ri(B, N), _s(0.03, dev), ri(B, N), _s(0.03, dev))


@pytest.mark.parametrize("s_dt,s_db", [(0.03, 0.05), (0.08, 0.02), (0.2, 0.1)])
@pytest.mark.parametrize("lanes", [4, 8])
def test_step_sizes_against_fp64_softplus(dev, s_dt, s_db, lanes):
    """The step size the forward kernels form, softplus(s_dt q + s_db q_b), read back through dt_sum_out on one-step
    sequences: every int8 code (one per batch entry) against 256 channels' biases, compared with the fp64 value.  The
    kernel's softplus is exp2 / log2 on the hardware with one compensated rounding; the arguments reach +-38."""
    import ctypes as ct
    from quamba_amd import _lib
    Bn, D, L, N = 256, 256, 1, 16
    q = torch.arange(-128, 128, dtype=torch.int8, device=dev).view(Bn, 1, 1).expand(Bn, D, L).contiguous()
    u = torch.ones(Bn, D, L, dtype=torch.int8, device=dev)
    A = torch.zeros(D, N, dtype=torch.int8, device=dev)
    Bm = torch.zeros(Bn, 1, N, L, dtype=torch.int8, device=dev)
    Cm = Bm.clone()
    db = torch.randint(-128, 128, (D,), dtype=torch.int8, device=dev, generator=torch.Generator(device=dev).manual_seed(3))
    out = torch.empty(Bn, L, D, dtype=torch.float16, device=dev)
    st = torch.empty(Bn, D, 1, N, dtype=torch.float32, device=dev)
    dts = torch.empty(Bn, D, dtype=torch.float32, device=dev)
    sc = [_s(v, dev) for v in (0.03, s_dt, 0.02, 0.03, 0.03, s_db)]
    p = _lib.QaSScanParams()
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups = Bn, D, L, N, 1
    p.delta_softplus = 1
    p.u_batch_stride, p.u_d_stride = u.stride(0), u.stride(1)
    p.delta_batch_stride, p.delta_d_stride = q.stride(0), q.stride(1)
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = Bm.stride(0), Bm.stride(1), Bm.stride(2)
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = Cm.stride(0), Cm.stride(1), Cm.stride(2)
    p.A_d_stride, p.A_dstate_stride = A.stride(0), A.stride(1)
    p.out_batch_stride, p.out_l_stride, p.out_d_stride = out.stride()
    p.u, p.delta, p.A_log, p.B, p.C, p.out = (t.data_ptr() for t in (u, q, A, Bm, Cm, out))
    p.scale_u, p.scale_delta, p.scale_A, p.scale_B, p.scale_C = (t.data_ptr() for t in sc[:5])
    p.delta_bias, p.scale_delta_bias = db.data_ptr(), sc[5].data_ptr()
    p.last_state_f32, p.dt_sum_out = st.data_ptr(), dts.data_ptr()
    p.mapping = ops.sscan_mapping(lanes, 4)
    _lib.check(_lib.lib().qa_sscan_fwd(ct.byref(p), _lib.current_stream(dev)), "sscan_fwd")
    torch.cuda.synchronize()
    x = (np.float32(s_dt) * np.arange(-128, 128, dtype=np.float32)[:, None]
         + np.float32(s_db) * db.cpu().numpy().astype(np.float32)[None, :])
    want = np.where(x > 20, x.astype(np.float64), np.log1p(np.exp(x.astype(np.float64))))
    got = dts.cpu().numpy().astype(np.float64)
    assert np.abs(got - want).max() > 0                       # hardware exp2 / log2: close, not equal
    assert (np.abs(got - want) / want).max() <= 1e-5


def test_module_forward_then_update_continue_the_same_sequence(dev):
    B, L, D, N = 2, 64, 96, 16
    d = synth.mamba1_scan_inputs(B, L + 4, D, N, seed=31)
    A_log = torch.from_numpy(d["A_log"].astype(np.float32) * d["s_A"]).to(dev)
    q = QSScan.from_fp16(N, D, A_log, D=torch.ones(D, device=dev),
                         dt_bias=torch.from_numpy(d["dt_bias"].astype(np.float32) * d["s_db"]).to(dev),
                         ssm_state_scale=torch.tensor(1.0), u_scale=torch.tensor(float(d["s_u"])),
                         dt_scale=torch.tensor(float(d["s_dt"])), B_scale=torch.tensor(float(d["s_B"])),
                         C_scale=torch.tensor(float(d["s_C"])), z_scale=torch.tensor(float(d["s_z"])))
    assert q.A_log.dtype == torch.int8 and q.A_log.shape == (D, N) and q.u_scale.dtype == torch.float32
    np.testing.assert_array_equal(q.A_log.cpu().numpy(), d["A_log"])
    full = {k: (v[..., :] if isinstance(v, np.ndarray) else v) for k, v in d.items()}
    y_all, _, _ = _oracle(full, 1.0)
    cut = lambda a: _t(a[:, :, :L], dev)
    y, state = q(cut(d["u"]), cut(d["dt"]), cut(d["B"]), cut(d["C"]), z=cut(d["z"]), return_last_state=True,
                 state_dtype=torch.float32)
    assert state.shape == (B, D, N)
    _check(y, y_all[:, :L])
    state = state.contiguous()
    for t in range(L, L + 4):
        yt, state = q.update(state, _t(d["u"][:, :, t], dev), _t(d["dt"][:, :, t], dev), _t(d["B"][:, :, t], dev),
                             _t(d["C"][:, :, t], dev), z=_t(d["z"][:, :, t], dev))
        np.testing.assert_allclose(yt.float().cpu().numpy(), y_all[:, t].astype(np.float16).astype(np.float32),
                                   rtol=RTOL, atol=ATOL)


def test_errors(dev):
    d = synth.mamba1_scan_inputs(1, 16, 8, 16, seed=1)
    args = lambda **o: dict(dict(u=_t(d["u"], dev), B=_t(d["B"][:, None], dev)), **o)
    with pytest.raises(NotImplementedError, match="input-dependent"):
        ops.sscan_fwd(_t(d["u"], dev), _s(1, dev), _t(d["dt"], dev), _s(1, dev), _t(d["A_log"], dev), _s(1, dev),
                      _t(d["B"][0], dev), _s(1, dev), _t(d["C"][0], dev), _s(1, dev), _s(1, dev))
    with pytest.raises(RuntimeError, match="int8"):
        ops.sscan_fwd(_t(d["u"], dev).float(), _s(1, dev), _t(d["dt"], dev), _s(1, dev), _t(d["A_log"], dev),
                      _s(1, dev), _t(d["B"][:, None], dev), _s(1, dev), _t(d["C"][:, None], dev), _s(1, dev), _s(1, dev))
    big_A = torch.zeros((8, 300), dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError, match="<= 256"):
        ops.sscan_fwd(_t(d["u"], dev), _s(1, dev), _t(d["dt"], dev), _s(1, dev), big_A, _s(1, dev),
                      _t(d["B"][:, None], dev), _s(1, dev), _t(d["C"][:, None], dev), _s(1, dev), _s(1, dev))


def test_mixed_launch_is_chosen_when_it_evens_out_the_waves(dev):
    """Batch 8 x 5120 channels is 2.5 waves per SIMD with four lanes per channel: the last fifth of the channels
    goes to the eight-lane kind.  Same answer as every channel with four lanes (the default for 4096 channels)."""
    B, L, D, N = 8, 96, 5120, 16
    g = torch.Generator(device=dev).manual_seed(3)
    ri = lambda *s: torch.randint(-128, 128, s, dtype=torch.int8, device=dev, generator=g)
    u, dt, z, Bm, Cm = ri(B, D, L), ri(B, D, L), ri(B, D, L), ri(B, 1, N, L), ri(B, 1, N, L)
    A, Dq, db = ri(D, N), ri(D), ri(D)
    s = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    run = lambda sl: ops.sscan_fwd(u[:, sl], s(0.03), dt[:, sl], s(0.02), A[sl], s(0.02), Bm, s(0.03), Cm, s(0.03), s(1.0), Dq[sl],
                                   s(0.008), z[:, sl], s(0.03), db[sl], s(0.01), True, state_dtype=torch.float32)
    y, st = run(slice(None))
    y_a, st_a = run(slice(0, 4096))
    y_b, st_b = run(slice(4096, 5120))
    np.testing.assert_allclose(y[:, :, :4096].float().cpu().numpy(), y_a.float().cpu().numpy(), rtol=1e-2, atol=1e-2)
    np.testing.assert_allclose(y[:, :, 4096:].float().cpu().numpy(), y_b.float().cpu().numpy(), rtol=1e-2, atol=1e-2)
    full = torch.cat([st_a, st_b], dim=1)
    assert float((st - full).abs().max()) <= 1e-3 * float(full.abs().max())

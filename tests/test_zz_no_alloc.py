"""The SSD chunk scan entry point that allocates nothing (qa_ssd_chunk_scan_fwd_noalloc: the intermediates live in
a fixed buffer inside the library's device image) against the entry point that takes a caller's workspace: same
kernels, so the fp16 outputs and the final states must be the same bits.  Two calls in a row share the buffer, the
second on a smaller input, so that whatever the first call left behind is in the way of the second."""
import ctypes as ct

import numpy as np
import pytest
import torch

from quamba_amd import _lib, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev):
    return None if a is None else torch.from_numpy(np.ascontiguousarray(a)).to(dev)


def _run(d, dev, chunk, state_scale, static):
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    return ops.ssd_chunk_scan_combined_fwd(
        _t(d["x"], dev), s(d["x_scale"]), _t(d["dt"], dev), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
        _t(d["B"], dev), s(d["s_B"]), _t(d["C"], dev), s(d["s_C"]), s(state_scale), chunk,
        q_D=_t(d["D"], dev), D_scale=s(d["s_D"]), q_z=_t(d["z"], dev), z_scale=s(d["s_z"]), dt_bias=_t(d["dt_bias"], dev),
        dt_softplus=True, x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev),
        final_state_dtype=torch.int8, static_scratch=static)


def test_two_calls_in_a_row_match_the_entry_point_with_a_workspace(dev):
    # batch, seqlen, heads, d_state, groups, chunk: the second problem is smaller in every dimension
    for B, L, H, N, G, Q in ((2, 300, 16, 128, 2, 128), (1, 89, 8, 64, 2, 64)):
        d = synth.mamba2_ssd_inputs(B, L, H, 64, N, G, seed=L, grouped=True, nhead_groups=4, ndim_groups=4, with_z=True)
        scale = np.full((G, 4, 4, N), 0.05, np.float32)
        y_ws, f_ws = _run(d, dev, Q, scale, static=False)
        y_st, f_st = _run(d, dev, Q, scale, static=True)
        torch.cuda.synchronize()
        assert y_st.dtype == torch.float16 and f_st.dtype == torch.int8
        assert torch.equal(y_st, y_ws) and torch.equal(f_st, f_ws)
        assert float(y_ws.float().abs().max()) > 1.0 and int(f_ws.abs().max()) > 10


def test_a_repeated_call_leaves_the_free_device_memory_unchanged(dev):
    """After one call (which also looks the buffer's address up and raises the kernels' LDS limit) a second call on
    the same shapes takes nothing from the device: torch serves the outputs from blocks it already holds, and the
    library itself allocates nothing, so the driver reports the same free bytes before and after."""
    d = synth.mamba2_ssd_inputs(2, 300, 16, 64, 128, 2, seed=5, grouped=True, nhead_groups=4, ndim_groups=4, with_z=True)
    scale = np.full((2, 4, 4, 128), 0.05, np.float32)
    y0, f0 = _run(d, dev, 128, scale, static=True)
    y0, f0 = y0.clone(), f0.clone()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    y1, f1 = _run(d, dev, 128, scale, static=True)
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(y1, y0) and torch.equal(f1, f0)


def test_capture_into_a_graph_after_one_warm_up_call(dev):
    """The first call on a device runs hipGetSymbolAddress and hipFuncSetAttribute, which do not belong under stream
    capture: one ordinary call comes first, then the entry point may be captured.  The graph is replayed three times
    with eager work and synchronisations in between, every replay against the eager result."""
    d = synth.mamba2_ssd_inputs(1, 200, 8, 64, 64, 1, seed=9, grouped=True, nhead_groups=2, ndim_groups=2, with_z=True)
    scale = np.full((1, 2, 2, 64), 0.05, np.float32)
    y_eager, f_eager = _run(d, dev, 64, scale, static=True)            # the warm-up call
    y_eager, f_eager = y_eager.clone(), f_eager.clone()
    torch.cuda.synchronize()
    # device-resident arguments built before the capture (a host-to-device copy cannot be captured)
    s = lambda v: torch.tensor(np.asarray(v, np.float32)).to(dev)
    args = (_t(d["x"], dev), s(d["x_scale"]), _t(d["dt"], dev), s(d["s_dt"]), _t(d["A_log"], dev), s(d["s_A"]),
            _t(d["B"], dev), s(d["s_B"]), _t(d["C"], dev), s(d["s_C"]), s(scale), 64)
    kw = dict(q_D=_t(d["D"], dev), D_scale=s(d["s_D"]), q_z=_t(d["z"], dev), z_scale=s(d["s_z"]), dt_bias=_t(d["dt_bias"], dev),
              dt_softplus=True, x_head_group_range=_t(d["head_range"], dev), x_dim_group_range=_t(d["dim_range"], dev),
              final_state_dtype=torch.int8, static_scratch=True)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_g, f_g = ops.ssd_chunk_scan_combined_fwd(*args, **kw)
    for rep in range(3):
        y_g.zero_(); f_g.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y_g, y_eager) and torch.equal(f_g, f_eager), f"replay {rep}"
        # eager work on the same buffer between the replays: another problem through the same entry point
        _run(synth.mamba2_ssd_inputs(1, 89, 8, 64, 64, 2, seed=rep, grouped=True, nhead_groups=4, ndim_groups=4, with_z=True),
             dev, 64, np.full((2, 4, 4, 64), 0.05, np.float32), static=True)
        torch.cuda.synchronize()


def test_sizes_beyond_the_fixed_buffer_are_refused(dev):
    # 4 x 4096 steps x 80 heads x 128 states needs 84 MB of intermediates, more than the 64 MiB the library holds: a clear
    # error, nothing launched.  Every operand is a real device tensor of the right size.
    B, L, H, N, Q = 4, 4096, 80, 128, 256
    z8 = lambda *shape: torch.zeros(shape, dtype=torch.int8, device=dev)
    one = torch.ones(1, dtype=torch.float32, device=dev)
    x, dt, A, Bm, Cm = z8(B, L, H, 64), torch.zeros(B, L, H, device=dev), z8(H), z8(B, L, 1, N), z8(B, L, 1, N)
    out, final = torch.empty(B, L, H, 64, dtype=torch.float16, device=dev), torch.empty(B, H, 64, N, device=dev)
    p = _lib.QaSsdParams()
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups, p.chunk_size = B, L, H, 64, N, 1, Q
    p.dt_is_fp32 = 1
    p.final_state_is_fp32 = 1
    p.x, p.dt, p.A_log, p.B, p.C, p.out, p.final_states = (t.data_ptr() for t in (x, dt, A, Bm, Cm, out, final))
    p.x_scale = p.A_log_scale = p.B_scale = p.C_scale = one.data_ptr()
    assert _lib.lib().qa_ssd_workspace_bytes(ct.byref(p)) > (64 << 20)
    st = _lib.lib().qa_ssd_chunk_scan_fwd_noalloc(ct.byref(p), None)
    torch.cuda.synchronize()
    assert st == -6
    with pytest.raises(RuntimeError, match="scratch"):
        _lib.check(st, "ssd_chunk_scan_fwd_noalloc")

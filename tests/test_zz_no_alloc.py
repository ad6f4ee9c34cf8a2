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


def test_sizes_beyond_the_fixed_buffer_are_refused(dev):
    # 4 x 4096 x 80 heads needs more than the 64 MiB the library holds: a clear error, nothing launched
    p = _lib.QaSsdParams()
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups, p.chunk_size = 8, 8192, 80, 64, 128, 1, 256
    p.dt_is_fp32 = 1
    p.final_state_is_fp32 = 1
    for name in ("x", "dt", "A_log", "B", "C", "out", "x_scale", "A_log_scale", "B_scale", "C_scale"):
        setattr(p, name, 256)                      # never dereferenced: the size check comes first
    assert _lib.lib().qa_ssd_workspace_bytes(ct.byref(p)) > (64 << 20)
    st = _lib.lib().qa_ssd_chunk_scan_fwd_noalloc(ct.byref(p), None)
    assert st == -6
    with pytest.raises(RuntimeError, match="scratch"):
        _lib.check(st, "ssd_chunk_scan_fwd_noalloc")

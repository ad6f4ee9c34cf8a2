"""GPU parity of the Mamba2 xBC conv (forward and update) against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import Quamb2Conv1D, ops, synth

pytestmark = pytest.mark.gpu


def _t(a, dev, dtype=None):
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    return t if dtype is None else t.to(dtype)


def _case(batch, seqlen, nheads, headdim, dstate, ngroups, **kw):
    c = synth.mamba2_conv_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, **kw)
    c.update(headdim=headdim, dstate=dstate, ngroups=ngroups)
    c["chan"] = oracle.quamba2_conv_channel_scales(
        c["x_dim"], headdim, dstate, ngroups, c["scales_in"], c["scales_w"], c["scales_b"], c["x_out_scales"],
        c["B_out_scales"], c["C_out_scales"], c["x_head_group_range"], c["x_dim_group_range"])
    return c


def _module(c, dev):
    grouped = c["x_head_group_range"] is not None
    nhg, ndg = (c["x_dim_group_range"].shape[1:] if grouped else (0, 0))
    m = Quamb2Conv1D(c["x_dim"], c["headdim"], c["dstate"], c["ngroups"], nhg, ndg, c["dim"], c["dim"],
                     c["weight"].shape[1], groups=c["dim"], bias=True if c["bias"] is not None else None, device=dev)
    m.weight = _t(c["weight"], dev)
    if c["bias"] is not None:
        m.bias = _t(c["bias"], dev)
        m.bx_scale, m.bB_scale, m.bC_scale = (float(v) for v in c["scales_b"])
    m.x_scale, m.B_scale, m.C_scale = (float(v) for v in c["scales_in"])
    m.wx_scale, m.wB_scale, m.wC_scale = (float(v) for v in c["scales_w"])
    m.x_out_scales = _t(c["x_out_scales"], dev)
    m.B_out_scales = _t(c["B_out_scales"], dev)
    m.C_out_scales = _t(c["C_out_scales"], dev)
    if grouped:
        m.x_head_group_range = _t(c["x_head_group_range"], dev)
        m.x_dim_group_range = _t(c["x_dim_group_range"], dev)
    return m


def _channel_last(q, dev):
    """(B, D, L) numpy -> torch view of the same shape over (B, L, D) memory."""
    return _t(np.ascontiguousarray(q.transpose(0, 2, 1)), dev).transpose(1, 2)


# (batch, seqlen, nheads, headdim, dstate, ngroups, grouped): model-like, ragged lengths, one group / several
CASES = [(2, 256, 16, 64, 128, 1, True), (1, 77, 8, 64, 128, 2, True), (3, 1, 4, 32, 64, 2, True),
         (2, 130, 8, 64, 128, 1, False), (1, 2051, 4, 64, 64, 4, True), (2, 33, 24, 64, 128, 8, True)]


@pytest.mark.parametrize("batch,seqlen,nheads,headdim,dstate,ngroups,grouped", CASES)
def test_fwd_bit_exact(dev, batch, seqlen, nheads, headdim, dstate, ngroups, grouped):
    c = _case(batch, seqlen, nheads, headdim, dstate, ngroups, grouped=grouped, seed=seqlen + nheads)
    want = oracle.quamba2_conv1d_fwd(c["xBC"], c["weight"], c["bias"], *c["chan"], c["x_dim"], c["bc"])
    m = _module(c, dev)
    got = m(_channel_last(c["xBC"], dev))
    for g, w, n in zip(got, want, (c["x_dim"], c["bc"], c["bc"])):
        assert g.shape == (batch, n, seqlen) and g.dtype == torch.int8
        assert g.stride(1) == 1 or n == 1                      # channel-contiguous, as the SSD kernel reads it
        np.testing.assert_array_equal(g.cpu().numpy(), w)
    assert max(int(np.abs(w).max()) for w in want) > 100       # the scales put the outputs on the full int8 range


def test_fwd_on_in_proj_slice(dev):
    # xBC as the mixer passes it: a channel slice of in_proj's (batch, seqlen, d_in_proj) output
    c = _case(2, 96, 8, 64, 128, 1, seed=7)
    d_inner, dim = c["x_dim"], c["dim"]
    buf = torch.zeros((2, 96, d_inner + dim + 8), dtype=torch.int8, device=dev)
    buf[:, :, d_inner:d_inner + dim] = _t(np.ascontiguousarray(c["xBC"].transpose(0, 2, 1)), dev)
    xBC = buf[:, :, d_inner:d_inner + dim].transpose(1, 2)
    want = oracle.quamba2_conv1d_fwd(c["xBC"], c["weight"], c["bias"], *c["chan"], c["x_dim"], c["bc"])
    got = _module(c, dev)(xBC)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)


def test_fwd_unaligned_takes_the_generic_kernel(dev):
    c = _case(1, 50, 4, 32, 64, 1, seed=9)
    buf = torch.zeros((1, 50, c["dim"] + 3), dtype=torch.int8, device=dev)
    buf[:, :, 1:1 + c["dim"]] = _t(np.ascontiguousarray(c["xBC"].transpose(0, 2, 1)), dev)
    xBC = buf[:, :, 1:1 + c["dim"]].transpose(1, 2)            # odd byte offset, odd row pitch
    want = oracle.quamba2_conv1d_fwd(c["xBC"], c["weight"], c["bias"], *c["chan"], c["x_dim"], c["bc"])
    got = _module(c, dev)(xBC)
    for g, w in zip(got, want):
        np.testing.assert_array_equal(g.cpu().numpy(), w)


@pytest.mark.parametrize("state_len", [4, 3])
@pytest.mark.parametrize("grouped", [True, False])
def test_update_bit_exact_and_state_in_place(dev, state_len, grouped):
    c = _case(3, 6, 8, 64, 128, 2, grouped=grouped, seed=21)
    m = _module(c, dev)
    g = np.random.default_rng(1)
    state = g.integers(-128, 128, (3, c["dim"], state_len)).astype(np.int8)
    dstate = _t(state, dev)
    for t in range(c["xBC"].shape[2]):
        step = np.ascontiguousarray(c["xBC"][:, :, t])
        wx, wB, wC, state = oracle.quamba2_conv1d_update(step, state, c["weight"], c["bias"], *c["chan"], c["x_dim"], c["bc"])
        gx, gB, gC = m.update(_t(step, dev), dstate)
        np.testing.assert_array_equal(gx.cpu().numpy(), wx)
        np.testing.assert_array_equal(gB.cpu().numpy(), wB)
        np.testing.assert_array_equal(gC.cpu().numpy(), wC)
        np.testing.assert_array_equal(dstate.cpu().numpy(), state)


def test_rejects_what_the_reference_rejects(dev):
    c = _case(1, 8, 4, 32, 64, 1, seed=2)
    m = _module(c, dev)
    with pytest.raises(RuntimeError):
        m(_t(c["xBC"], dev))                                   # seqlen-contiguous input
    with pytest.raises(RuntimeError):
        ops.quamba2_conv1d_fwd(_channel_last(c["xBC"], dev), 1.0, 1.0, 1.0, c["x_dim"] - 32, 32, 64, 1, None, None,
                               m.x_out_scales[:1].reshape(1), m.B_out_scales, m.C_out_scales, m.weight, 1.0, 1.0, 1.0)
    with pytest.raises(NotImplementedError):
        ops.quamba2_conv1d_fwd(_channel_last(c["xBC"], dev), *m._args()[:-4], torch.zeros(1), None, None, True)


def test_state_dict_round_trip(dev):
    c = _case(1, 8, 4, 32, 64, 2, seed=4)
    m = _module(c, dev)
    sd = m.state_dict()
    for k in ("x_scale", "wB_scale", "bC_scale", "weight", "bias", "x_out_scales", "x_head_group_range"):
        assert k in sd
    m2 = Quamb2Conv1D(c["x_dim"], 32, 64, 2, *c["x_dim_group_range"].shape[1:], c["dim"], c["dim"], 4, groups=c["dim"],
                      device=dev)
    m2.load_state_dict(sd)
    x = _channel_last(c["xBC"], dev)
    for a, b in zip(m(x), m2(x)):
        assert torch.equal(a, b)

"""Pins the CPU oracle's Mamba2 xBC conv restatement (no GPU): with one scale everywhere it must equal the
(separately pinned) Mamba1 conv restatement, the group-range walk is checked against a searchsorted
formulation, the dequantised result against torch's conv1d, and forward against update iterated."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from quamba_amd import synth


def _scales(c):
    return oracle.quamba2_conv_channel_scales(
        c["x_dim"], c["headdim"], c["dstate"], c["ngroups"], c["scales_in"], c["scales_w"], c["scales_b"],
        c["x_out_scales"], c["B_out_scales"], c["C_out_scales"], c["x_head_group_range"], c["x_dim_group_range"])


def _case(batch=2, seqlen=37, nheads=8, headdim=16, dstate=32, ngroups=2, **kw):
    c = synth.mamba2_conv_inputs(batch, seqlen, nheads, headdim, dstate, ngroups, **kw)
    c.update(headdim=headdim, dstate=dstate, ngroups=ngroups, nheads=nheads)
    return c


def test_uniform_scales_reduce_to_the_mamba1_conv():
    c = _case(grouped=False)
    s_x, s_w, s_b, s_o = np.float32(0.03), np.float32(0.004), np.float32(0.002), np.float32(0.05)
    dim = c["dim"]
    full = lambda v: np.full(dim, v, np.float32)
    x, B, C = oracle.quamba2_conv1d_fwd(c["xBC"], c["weight"], c["bias"], full(s_w * s_x), full(s_b), full(s_o),
                                         c["x_dim"], c["bc"])
    want = oracle.conv1d_fwd(c["xBC"], c["weight"], c["bias"], s_x, s_w, s_b, s_o, silu=True, tapwise=False)
    np.testing.assert_array_equal(np.concatenate([x, B, C], axis=1), want)


@pytest.mark.parametrize("ngroups,nhg,ndg", [(1, 4, 4), (2, 3, 5), (4, 2, 1), (2, 1, 3)])
def test_group_range_walk_matches_searchsorted(ngroups, nhg, ndg):
    c = _case(nheads=16, headdim=16, dstate=16, ngroups=ngroups, nhead_groups=nhg, ndim_groups=ndg, seed=ngroups + nhg)
    s_in, s_bias, s_out = _scales(c)
    x_dim, hd, ds = c["x_dim"], c["headdim"], c["dstate"]
    hpg = c["nheads"] // ngroups
    hr, dr, xs = c["x_head_group_range"], c["x_dim_group_range"], c["x_out_scales"]
    for ch in range(c["dim"]):
        if ch < x_dim:
            g, head, d = ch // (hpg * hd), (ch // hd) % hpg, ch % hd
            hg = int(np.searchsorted(hr[g], head, side="right"))
            dg = int(np.searchsorted(dr[g, hg], d, side="right"))
            assert s_out[ch] == xs[g, hg, dg]
            assert s_in[ch] == np.float32(c["scales_w"][0]) * np.float32(c["scales_in"][0])
        elif ch < x_dim + c["bc"]:
            assert s_out[ch] == c["B_out_scales"][(ch - x_dim) // ds]
            assert s_bias[ch] == np.float32(c["scales_b"][1])
        else:
            assert s_out[ch] == c["C_out_scales"][(ch - x_dim - c["bc"]) // ds]
            assert s_in[ch] == np.float32(c["scales_w"][2]) * np.float32(c["scales_in"][2])
    # every group cell is used by at least one channel
    assert set(np.unique(s_out[:x_dim])) == set(np.unique(xs))


@pytest.mark.parametrize("grouped", [True, False])
def test_dequantised_output_matches_torch_conv1d(grouped):
    c = _case(batch=2, seqlen=64, grouped=grouped)
    s_in, s_bias, s_out = _scales(c)
    x, B, C = oracle.quamba2_conv1d_fwd(c["xBC"], c["weight"], c["bias"], s_in, s_bias, s_out, c["x_dim"], c["bc"])
    got = np.concatenate([x, B, C], axis=1).astype(np.float64) * s_out[None, :, None]
    # library routine: per-channel dequantised taps and inputs through torch's depthwise conv1d in float64
    dim, k = c["weight"].shape
    x_scale = np.concatenate([np.full(n, s, np.float64) for n, s in zip((c["x_dim"], c["bc"], c["bc"]), c["scales_in"])])
    w_scale = np.concatenate([np.full(n, s, np.float64) for n, s in zip((c["x_dim"], c["bc"], c["bc"]), c["scales_w"])])
    xf = torch.from_numpy(c["xBC"].astype(np.float64) * x_scale[None, :, None])
    wf = torch.from_numpy(c["weight"].astype(np.float64) * w_scale[:, None]).unsqueeze(1)
    bf = torch.from_numpy(c["bias"].astype(np.float64) * s_bias.astype(np.float64))
    want = F.silu(F.conv1d(xf, wf, bf, padding=k - 1, groups=dim)[..., :xf.shape[-1]]).numpy()
    # one rounding step of the output grid, except where the value saturates
    err = np.abs(got - want)
    sat = np.abs(want) >= 127 * s_out[None, :, None]
    assert np.all((err <= 0.5001 * s_out[None, :, None] + 1e-6) | sat)


@pytest.mark.parametrize("state_len", [4, 3])
def test_forward_equals_update_iterated_on_unit_weights(state_len):
    # with taps in {-1, 0, 1} and no bias both op orders are exact, so the two paths must agree bit for bit
    c = _case(batch=2, seqlen=19, bias=False)
    g = np.random.default_rng(3)
    w = g.integers(-1, 2, c["weight"].shape).astype(np.int8)
    s_in, s_bias, s_out = _scales(c)
    s_in = np.full_like(s_in, 2.0 ** -6)            # power of two: products stay exact
    x, B, C = oracle.quamba2_conv1d_fwd(c["xBC"], w, None, s_in, s_bias, s_out, c["x_dim"], c["bc"], silu=False)
    state = np.zeros((2, c["dim"], state_len), np.int8)
    for t in range(c["xBC"].shape[2]):
        xs, Bs, Cs, state = oracle.quamba2_conv1d_update(np.ascontiguousarray(c["xBC"][:, :, t]), state, w, None,
                                                          s_in, s_bias, s_out, c["x_dim"], c["bc"], silu=False)
        np.testing.assert_array_equal(xs, x[:, :, t])
        np.testing.assert_array_equal(Bs, B[:, :, t])
        np.testing.assert_array_equal(Cs, C[:, :, t])
    np.testing.assert_array_equal(state[:, :, -3:], c["xBC"][:, :, -3:])

"""GPU parity of the int8 causal conv1d (forward and update) against the CPU oracle: bit-exact."""
import numpy as np
import pytest
import torch

import oracle
from quamba_amd import QCausalConv1D, ops, synth

pytestmark = pytest.mark.gpu


def _case(B, D, L, k, seed, bias=True):
    qx, sx = synth.quantize_absmax(synth.activations((B, D, L), 1, seed, "x"))
    qw, sw, qb, sb = synth.conv_weights(D, k, seed, bias=bias)
    so = synth.conv_output_scale(qx, sx, qw, sw, qb, sb)
    return qx, sx, qw, sw, qb, sb, so


def _t(a, dev):
    return None if a is None else torch.from_numpy(a).to(dev)


# (batch, dim, seqlen, width): model-shaped rows plus ragged and tiny lengths
SHAPES = [(1, 1536, 512, 4), (2, 1536, 33, 4), (3, 64, 1, 4), (2, 48, 17, 3), (2, 40, 100, 2),
          (1, 5120, 1024, 4), (2, 24, 2048 + 5, 4)]


@pytest.mark.parametrize("B,D,L,k", SHAPES)
@pytest.mark.parametrize("silu", [True, False])
def test_fwd_seqlen_contiguous_bit_exact(dev, B, D, L, k, silu):
    qx, sx, qw, sw, qb, sb, so = _case(B, D, L, k, seed=L + D)
    want = oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so, silu=silu)
    got = ops.causal_conv1d_fwd(_t(qx, dev), sx, _t(qw, dev), sw, so, sb, _t(qb, dev), None, None, None, silu)
    assert got.shape == (B, D, L) and got.dtype == torch.int8
    np.testing.assert_array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("s_in,s_out", [(0.02, 0.02), (0.004, 0.001), (0.3, 0.05), (0.05, 2.0), (0.01, 1e-5), (0.0002, 2e-7)])
def test_fwd_bit_exact_over_wide_ranges_of_the_pre_activation(dev, s_in, s_out):
    """Uniform int8 inputs and taps: the accumulator sweeps +-65000, so with these scales the SiLU argument
    covers fractions of a unit up to several hundred units either side of zero, and the outputs run from
    all-saturated to all-zero.  Two million outputs per case land on every side of the rounding margins of
    the fast epilogue and of its switch to the exact route for very negative arguments."""
    g = np.random.default_rng(int(s_in * 1e4) + 7)
    B, D, L = 2, 256, 4096
    qx = g.integers(-128, 128, (B, D, L)).astype(np.int8)
    qw = g.integers(-128, 128, (D, 4)).astype(np.int8)
    qb = g.integers(-128, 128, D).astype(np.int8)
    sw, sb = 0.01, 0.02
    want = oracle.conv1d_fwd(qx, qw, qb, s_in, sw, sb, s_out)
    got = ops.causal_conv1d_fwd(_t(qx, dev), s_in, _t(qw, dev), sw, s_out, sb, _t(qb, dev))
    np.testing.assert_array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("s_out", [0.1, 0.03, 0.0031, 0.0025, 0.0024, 0.0007])
def test_fwd_bit_exact_with_unsaturated_outputs_on_both_sides_of_the_margin_switch(dev, s_out):
    """Small taps keep the accumulator within +-4100, and the input scale is chosen so that the requantised value
    spans about +-150 codes: nearly all of the two million outputs are unsaturated, with up to a million distinct
    pre-activation values, so thousands of them fall inside the fast epilogue's rounding margin and next to it.  The
    output scales straddle 2.5e-3, where the margin changes from 1.25e-4 to 5e-4 of a code."""
    g = np.random.default_rng(int(s_out * 1e5) + 3)
    B, D, L = 2, 256, 4096
    qx = g.integers(-128, 128, (B, D, L)).astype(np.int8)
    qw = g.integers(-8, 9, (D, 4)).astype(np.int8)
    qb = g.integers(-128, 128, D).astype(np.int8)
    sw = 0.01
    s_in = 150.0 * s_out / (4100 * sw)
    sb = 20.0 * s_out / 128
    for silu in (True, False):
        want = oracle.conv1d_fwd(qx, qw, qb, s_in, sw, sb, s_out, silu=silu)
        assert np.mean(np.abs(want.astype(np.int32)) < 127) > 0.9
        got = ops.causal_conv1d_fwd(_t(qx, dev), s_in, _t(qw, dev), sw, s_out, sb, _t(qb, dev), None, None, None, silu)
        np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_fwd_no_bias(dev):
    qx, sx, qw, sw, qb, sb, so = _case(2, 128, 256, 4, seed=5, bias=False)
    want = oracle.conv1d_fwd(qx, qw, None, sx, sw, sb, so)
    got = ops.causal_conv1d_fwd(_t(qx, dev), sx, _t(qw, dev), sw, so, sb, None)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


def test_fwd_on_in_proj_view(dev):
    # the layout the mixer really feeds: x is the first half of a [2D][B][L] buffer viewed (B, D, L)
    B, D, L, k = 4, 256, 512, 4
    qx, sx, qw, sw, qb, sb, so = _case(B, D, L, k, seed=11)
    buf = torch.zeros((2 * D, B, L), dtype=torch.int8, device=dev)
    xz = buf.transpose(0, 1)                    # (B, 2D, L), strides (L, B*L, 1)
    x = xz[:, :D]
    x.copy_(_t(qx, dev))
    assert x.stride() == (L, B * L, 1)
    got = ops.causal_conv1d_fwd(x, sx, _t(qw, dev), sw, so, sb, _t(qb, dev))
    assert got.stride() == x.stride()
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so))


@pytest.mark.parametrize("B,D,L", [(5, 70, 2048), (7, 64, 96), (3, 33, 2064), (8, 130, 4096), (6, 20, 100)])
def test_fwd_on_in_proj_view_with_odd_batches_and_channel_counts(dev, B, D, L):
    """The (B, D, L) view of a [2D][B][L] buffer with batch sizes that do not fill a workgroup of four batch entries,
    channel counts that leave the bias vector without whole words, rows of two segments per lane and ragged rows."""
    qx, sx, qw, sw, qb, sb, so = _case(B, D, L, 4, seed=B * 1000 + D)
    buf = torch.zeros((2 * D, B, L), dtype=torch.int8, device=dev)
    x = buf.transpose(0, 1)[:, :D]
    x.copy_(_t(qx, dev))
    got = ops.causal_conv1d_fwd(x, sx, _t(qw, dev), sw, so, sb, _t(qb, dev))
    assert got.stride() == x.stride()
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so))


def test_fwd_unaligned_rows_take_the_generic_path(dev):
    B, D, L, k = 2, 32, 50, 4                   # row stride 50 is not a multiple of 16
    qx, sx, qw, sw, qb, sb, so = _case(B, D, L, k, seed=13)
    got = ops.causal_conv1d_fwd(_t(qx, dev), sx, _t(qw, dev), sw, so, sb, _t(qb, dev))
    np.testing.assert_array_equal(got.cpu().numpy(), oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so))


def test_fwd_channel_contiguous(dev):
    B, D, L, k = 2, 64, 96, 4
    qx, sx, qw, sw, qb, sb, so = _case(B, D, L, k, seed=17)
    x = _t(np.ascontiguousarray(qx.transpose(0, 2, 1)), dev).transpose(1, 2)   # (B, D, L), stride(1) == 1
    assert x.stride(1) == 1
    got = ops.causal_conv1d_fwd(x, sx, _t(qw, dev), sw, so, sb, _t(qb, dev))
    want = oracle.conv1d_fwd(qx, qw, qb, sx, sw, sb, so, tapwise=True)
    np.testing.assert_array_equal(got.cpu().numpy(), want)


@pytest.mark.parametrize("B,D,k,slen", [(1, 1536, 4, 4), (64, 5120, 4, 3), (16, 100, 3, 3), (5, 77, 2, 1)])
def test_update_bit_exact_and_state_in_place(dev, B, D, k, slen):
    steps = 6
    qx, sx, qw, sw, qb, sb, so = _case(B, D, steps, k, seed=D + k)
    state_ref = np.random.default_rng(D).integers(-128, 128, (B, D, slen)).astype(np.int8)
    state = _t(state_ref.copy(), dev)
    w, b = _t(qw, dev), _t(qb, dev)
    for t in range(steps):
        want, state_ref = oracle.conv1d_update(qx[:, :, t], state_ref, qw, qb, sx, sw, sb, so)
        got = ops.causal_conv1d_update(_t(np.ascontiguousarray(qx[:, :, t]), dev), state, sx, w, sw, so, sb, b)
        np.testing.assert_array_equal(got.cpu().numpy(), want)
        np.testing.assert_array_equal(state.cpu().numpy(), state_ref)


def test_module_surface(dev):
    conv = torch.nn.Conv1d(96, 96, 4, groups=96, padding=3, bias=True)
    q = QCausalConv1D.from_fp16(conv, input_scale=0.05, output_scale=0.02).to(dev)
    assert q.weight.shape == (96, 4) and q.weight.dtype == torch.int8 and q.bias.dtype == torch.int8
    sd = q.state_dict()
    assert {"weight", "bias", "weight_scale", "bias_scale", "input_scale", "output_scale"} <= set(sd)
    q2 = QCausalConv1D(96, 96, 4, groups=96, device=dev)
    q2.load_state_dict(sd)
    assert q2.input_scale == pytest.approx(0.05) and q2.weight_scale == pytest.approx(q.weight_scale)
    x = torch.randint(-128, 128, (2, 96, 64), dtype=torch.int8, device=dev)
    y = q2(x)
    want = oracle.conv1d_fwd(x.cpu().numpy(), q.weight.cpu().numpy(), q.bias.cpu().numpy(),
                             0.05, q.weight_scale, q.bias_scale, 0.02)
    np.testing.assert_array_equal(y.cpu().numpy(), want)
    state = torch.zeros((2, 96, 4), dtype=torch.int8, device=dev)
    for t in range(8):
        yt = q2.update(x[:, :, t].contiguous(), state)
    # after 8 steps the rolling state holds the last four inputs
    np.testing.assert_array_equal(state.cpu().numpy(), x[:, :, 4:8].cpu().numpy())
    assert yt.shape == (2, 96)


def test_errors(dev):
    x = torch.zeros((1, 8, 16), dtype=torch.int8, device=dev)
    w5 = torch.zeros((8, 5), dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError, match="width between 2 and 4"):
        ops.causal_conv1d_fwd(x, 1.0, w5, 1.0, 1.0, 1.0)
    w = torch.zeros((8, 4), dtype=torch.int8, device=dev)
    with pytest.raises(RuntimeError, match="int8"):
        ops.causal_conv1d_fwd(x.float(), 1.0, w, 1.0, 1.0, 1.0)
    with pytest.raises(NotImplementedError):
        ops.causal_conv1d_fwd(x, 1.0, w, 1.0, 1.0, 1.0, None, torch.zeros(1, device=dev))
    with pytest.raises(RuntimeError, match="GPU"):
        ops.causal_conv1d_fwd(x.cpu(), 1.0, w, 1.0, 1.0, 1.0)


@pytest.mark.parametrize("B,D,L", [(2, 64, 64), (1, 96, 100), (3, 200, 333), (2, 5120, 256), (1, 48, 17)])
def test_second_output_with_channels_contiguous(dev, B, D, L):
    """The optional (batch, seqlen, dim) copy written by the same kernel equals the transposed first output, and
    the first output equals the oracle bit for bit (ragged tiles in both directions included)."""
    qx, sx = synth.quantize_absmax(synth.activations((B, D, L + (-L) % 16), 1, 7 + D, "x"))
    qw, sw, qb, sb = synth.conv_weights(D, 4, 11)
    so = synth.conv_output_scale(qx, sx, qw, sw, qb, sb)
    x = torch.from_numpy(qx).to(dev)[:, :, :L]               # rows stay 16-byte aligned, seqlen may be ragged
    out, out_t = ops.causal_conv1d_fwd(x, sx, torch.from_numpy(qw).to(dev), sw, so, sb, torch.from_numpy(qb).to(dev),
                                       also_channel_last=True)
    want = oracle.conv1d_fwd(np.ascontiguousarray(qx[:, :, :L]), qw, qb, sx, sw, sb, so)
    assert out_t.shape == (B, L, D) and out_t.is_contiguous()
    np.testing.assert_array_equal(out.cpu().numpy(), want)
    np.testing.assert_array_equal(out_t.cpu().numpy(), want.transpose(0, 2, 1))

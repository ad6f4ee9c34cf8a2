"""The W4A8 weight quantiser and the Marlin-QQQ reader/writer against vectors produced by the reference's own
pure-Python packer (tests/golden/marlin_qqq_w4a8.npz, written by tests/golden/make_marlin_qqq_fixture.py)."""
import os

import numpy as np
import pytest
import torch

from quamba_amd import w4a8_utils as U

FIX = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "marlin_qqq_w4a8.npz"))
T = lambda k: torch.from_numpy(FIX[k])


def test_permutations_match_the_reference():
    np.testing.assert_array_equal(U.marlin_qqq_weight_perm("per-group").numpy(), FIX["perm_group"])
    np.testing.assert_array_equal(U.marlin_qqq_weight_perm("per-channel").numpy(), FIX["perm_channel"])
    sp, sps = U.marlin_qqq_scale_perms()
    np.testing.assert_array_equal(sp.numpy(), FIX["scale_perm"])
    np.testing.assert_array_equal(sps.numpy(), FIX["scale_perm_single"])
    for p in (FIX["perm_group"], FIX["perm_channel"]):
        assert sorted(p.tolist()) == list(range(1024))


def test_group_quantiser_matches_the_reference_bit_for_bit():
    w_ref, q_w, s_group, s_channel = U.get_w4a8_quantize_weights(T("g_w").clone(), 4, 128)
    np.testing.assert_array_equal(q_w.numpy(), FIX["g_q_w"])
    np.testing.assert_array_equal(s_group.numpy(), FIX["g_s_group"])
    np.testing.assert_array_equal(s_channel.numpy(), FIX["g_s_channel"])
    np.testing.assert_array_equal(w_ref.numpy(), FIX["g_w_ref"])


def test_channel_quantiser_matches_the_reference_bit_for_bit():
    w_ref, q_w, s_group, s_channel = U.get_w4a8_quantize_weights(T("c_w").clone(), 4, -1)
    np.testing.assert_array_equal(q_w.numpy(), FIX["c_q_w"])
    np.testing.assert_array_equal(s_channel.numpy(), FIX["c_s_channel"])
    np.testing.assert_array_equal(w_ref.numpy(), FIX["c_w_ref"])
    assert s_group.numel() == 0


def test_pack_matches_the_reference_words():
    np.testing.assert_array_equal(U.marlin_qqq_pack(T("g_q_w"), 256, 128, 128).numpy(), FIX["g_marlin_q_w"])
    np.testing.assert_array_equal(U.marlin_qqq_pack(T("c_q_w"), 128, 64, -1).numpy(), FIX["c_marlin_q_w"])
    sg, sc = U.marlin_qqq_permute_scales(T("g_s_group"), T("g_s_channel"), 256, 128, 128)
    np.testing.assert_array_equal(sg.numpy(), FIX["g_marlin_s_group"])
    np.testing.assert_array_equal(sc.numpy(), FIX["g_marlin_s_channel"])
    _, sc = U.marlin_qqq_permute_scales(torch.tensor([]), T("c_s_channel"), 128, 64, -1)
    np.testing.assert_array_equal(sc.numpy(), FIX["c_marlin_s_channel"])


def test_unpack_inverts_the_reference_words():
    np.testing.assert_array_equal(U.marlin_qqq_unpack(T("g_marlin_q_w"), 256, 128, 128).numpy(), FIX["g_q_w"])
    np.testing.assert_array_equal(U.marlin_qqq_unpack(T("c_marlin_q_w"), 128, 64, -1).numpy(), FIX["c_q_w"] & 0xF)
    sg, sc = U.marlin_qqq_unpermute_scales(T("g_marlin_s_group"), T("g_marlin_s_channel"), 256, 128, 128)
    np.testing.assert_array_equal(sg.numpy(), FIX["g_s_group"])
    np.testing.assert_array_equal(sc.numpy(), FIX["g_s_channel"])


def test_to_native_equals_quantising_here():
    packed, sg, sc = U.marlin_qqq_to_native(T("g_marlin_q_w"), T("g_marlin_s_group"), T("g_marlin_s_channel"), 256, 128)
    _, want_packed, want_sg, want_sc = U.w4a8_quantize(T("g_w").clone(), 4, 128)
    assert torch.equal(packed, want_packed) and torch.equal(sg, want_sg) and torch.equal(sc, want_sc)
    packed, sg, sc = U.marlin_qqq_to_native(T("c_marlin_q_w"), torch.tensor([], dtype=torch.half), T("c_marlin_s_channel"), 128, 64)
    _, want_packed, want_sg, want_sc = U.w4a8_quantize(T("c_w").clone(), 4, -1)
    assert torch.equal(packed, want_packed) and torch.equal(sc, want_sc) and sg.shape == (0, 64)


def test_padded_layer_with_fused_output_scales():
    # 128 real columns + 64 padding columns; padding decodes to zero weights either way
    packed, sg, sc = U.marlin_qqq_to_native(T("gp_marlin_q_w"), T("gp_marlin_s_group"), T("gp_marlin_s_channel"), 256, 192)
    _, want_packed, want_sg, want_sc = U.w4a8_quantize(T("g_w").clone(), 4, 128, out_scales=T("g_out_scales"), pad_out=64)
    assert torch.equal(packed[:128], want_packed[:128])
    assert torch.equal(sg[:, :128], want_sg[:, :128]) and torch.equal(sc[:, :128], want_sc[:, :128])
    assert torch.all(sg[:, 128:] == 0) and torch.all(want_sg[:, 128:] == 0)


@pytest.mark.parametrize("K,N,g", [(256, 128, 128), (512, 192, 128), (128, 64, -1), (64, 256, -1)])
def test_round_trip_on_random_codes(K, N, g):
    codes = torch.randint(0, 16, (K, N), dtype=torch.int32, generator=torch.Generator().manual_seed(K + N))
    assert torch.equal(U.marlin_qqq_unpack(U.marlin_qqq_pack(codes, K, N, g), K, N, g), codes)
    sg = torch.randn(max(K // 128, 1), N).half() if g == 128 else torch.tensor([], dtype=torch.half)
    sc = torch.randn(1, N)
    psg, psc = U.marlin_qqq_permute_scales(sg, sc, K, N, g)
    usg, usc = U.marlin_qqq_unpermute_scales(psg, psc, K, N, g)
    assert torch.equal(usc, sc) and (g != 128 or torch.equal(usg, sg))

"""Offline 4-bit weight quantisation for the W4A8 linears and this library's weight packing.

Numerics follow quamba/marlin_utils.py:139-262 (``get_w4a8_quantize_weights`` / ``w4a8_quantize``):
group scale = 2 * max|w_group| / 15, code = clamp(round(w / s) + 8, 0, 15), second-level int8
channel scale = max_k |w_ref| / 127, fused fp16 group scale = s_group / s_channel; per-channel
mode: code = clamp(round(w / (max|w| / 7)), -7, 7) as a signed nibble, s_channel /= 16.
Only the storage differs: codes are packed for the gfx950 kernel (``pack_w4a8``) and the scales are
kept in natural column order (the reference permutes both for its tensor-core tiles).

The second half of the file reads and writes the reference's own storage (Marlin-QQQ, quamba/marlin_utils.py
:33-133) so that checkpoints made by the reference load here: ``marlin_qqq_to_native`` turns the packed
int32 weight and the permuted scales into this library's buffers, ``marlin_qqq_pack`` is the forward
direction (used to check the inverse against vectors produced by the reference's own packer).
"""
import numpy as np
import torch


def pack_w4a8(codes_kn):
    """(K, N) integer codes (low 4 bits used) -> uint8 (N, K/2).

    Each aligned group of 8 codes of a column becomes 4 bytes: byte i holds code[8w+i] in the low
    nibble and code[8w+4+i] in the high nibble.
    """
    K, N = codes_kn.shape
    assert K % 8 == 0
    c = (codes_kn.t().contiguous().to(torch.int32) & 0xF).reshape(N, K // 8, 2, 4)
    packed = c[:, :, 0, :] | (c[:, :, 1, :] << 4)
    return packed.reshape(N, K // 2).to(torch.uint8).contiguous()


def unpack_w4a8(packed_nk2):
    """Inverse of pack_w4a8: uint8 (N, K/2) -> int32 codes (K, N) in [0, 15]."""
    N, K2 = packed_nk2.shape
    p = packed_nk2.to(torch.int32).reshape(N, K2 // 4, 4)
    codes = torch.stack([p & 0xF, (p >> 4) & 0xF], dim=2)      # (N, words, 2, 4)
    return codes.reshape(N, K2 * 2).t().contiguous()


@torch.no_grad()
def get_w4a8_quantize_weights(w, num_bits=4, group_size=-1):
    """w: float (K, N).  Returns (w_ref (K,N) fp16, q_w (K,N) int32 codes, s_group fp16 (K/g, N) already
    divided by s_channel, s_channel fp32 (1, N))."""
    assert w.is_floating_point() and num_bits == 4
    size_k, size_n = w.shape
    if group_size == -1:
        group_size = size_k
    assert group_size in (128, size_k) and group_size <= size_k
    if group_size < size_k:
        max_q, half_q = 15, 8
        wg = w.reshape(-1, group_size, size_n)
        s_group = wg.abs().amax(dim=1, keepdim=True) * (2.0 / max_q)                 # (G, 1, N)
        q_w = torch.clamp(torch.round(wg / s_group).int() + half_q, 0, max_q)
        w_ref = ((q_w - half_q).half() * s_group).reshape(size_k, size_n)
        q_w = q_w.reshape(size_k, size_n)
        s_channel = w_ref.abs().amax(dim=0, keepdim=True) / 127.0
        t_int8 = (w_ref / s_channel).round().clamp(-128, 127).to(torch.int8)
        w_ref = t_int8.half() * s_channel
        s_channel = s_channel.reshape(1, -1).float()
        s_group = (s_group.reshape(-1, size_n) / s_channel).half()
    else:
        max_q = 7
        s_channel = w.abs().amax(dim=0, keepdim=True) / max_q
        q_w = torch.clamp(torch.round(w / s_channel).int(), -max_q, max_q)
        w_ref = q_w.half() * s_channel
        s_group = torch.tensor([], dtype=torch.half, device=w.device)
        s_channel = (s_channel / 16.0).reshape(-1, size_n).float()
    return w_ref, q_w, s_group, s_channel


@torch.no_grad()
def w4a8_quantize(w, num_bits=4, group_size=-1, s_group=None, s_channel=None, out_scales=None, pad_out=0):
    """Quantises (or, given GPTQ scales, re-encodes) w (K, N) and packs it.
    Returns [w_ref (K, N+pad), packed uint8 (N+pad, K/2), s_group fp16 (K/g, N+pad), s_channel fp32 (1, N+pad)]."""
    size_k, size_n = w.shape
    if group_size == -1:
        group_size = size_k
    assert group_size <= size_k
    if s_group is None or s_channel is None:
        w_ref, q_w, s_group, s_channel = get_w4a8_quantize_weights(w, num_bits, group_size)
    else:
        w_ref = w.clone()
        wg = w.reshape(-1, group_size, size_n)
        q_w = torch.clamp(((wg / s_group.unsqueeze(1)) + 8).round().int(), 0, 15).reshape(size_k, size_n)
        s_channel = s_channel.float()
        s_group = torch.nan_to_num((s_group.reshape(-1, size_n) / s_channel).half(), nan=0.0)
    if out_scales is not None:
        s_channel = s_channel / out_scales.to(s_channel.device).float()
    if pad_out:
        pad = torch.nn.functional.pad
        w_ref = pad(w_ref, (0, pad_out, 0, 0), "constant", 0)
        # padding columns decode to w8 = 0: code 8 (value 0) in grouped mode, 0 in per-channel mode
        q_w = pad(q_w, (0, pad_out, 0, 0), "constant", 8 if group_size < size_k else 0)
        if s_group.numel():
            s_group = pad(s_group, (0, pad_out), "constant", 0)
        s_channel = pad(s_channel, (0, pad_out), "constant", 1e-6)
    return [w_ref, pack_w4a8(q_w), s_group, s_channel]


# ---------------------------------------------------------------------------------------------
# Marlin-QQQ storage (the reference's checkpoints)
# ---------------------------------------------------------------------------------------------
def marlin_qqq_weight_perm(quant_type):
    """The 1024-entry gather that orders four 16x16 tiles for the reference's tensor-core fragments
    (quamba/marlin_utils.py:71-105).  Output position (i, j, e), i < 32 a fragment lane, j < 4 the tile,
    e < 8 the nibble slot, reads flat tile element 256*j + 16*row + col with row = 4*(i % 4) + e % 4 and
    col = i // 4 + 8*(e // 4); the eight slots of a word are then interleaved so that the kernel's
    nibble extraction yields consecutive values (a different interleave for the per-channel scheme)."""
    assert quant_type in ("per-channel", "per-group"), "not supported quantization type"
    i = np.arange(32).reshape(32, 1, 1)
    j = np.arange(4).reshape(1, 4, 1)
    e = np.arange(8).reshape(1, 1, 8)
    src = 256 * j + 16 * (4 * (i % 4) + e % 4) + i // 4 + 8 * (e // 4)
    order = [4, 0, 5, 1, 6, 2, 7, 3] if quant_type == "per-channel" else [0, 2, 4, 6, 1, 3, 5, 7]
    return torch.from_numpy(src[:, :, order].reshape(-1).astype(np.int64))


def marlin_qqq_scale_perms():
    """(group-scale permutation over 64 columns: an 8x8 transposition; channel-scale permutation over
    32 columns) of quamba/marlin_utils.py:108-118."""
    i = np.arange(8).reshape(8, 1)
    scale_perm = (i + 8 * np.arange(8).reshape(1, 8)).reshape(-1)
    offs = np.array([0, 1, 8, 9, 16, 17, 24, 25])
    single = (2 * np.arange(4).reshape(4, 1) + offs.reshape(1, 8)).reshape(-1)
    return torch.from_numpy(scale_perm.astype(np.int64)), torch.from_numpy(single.astype(np.int64))


def _tile_rows(q_w, size_k, size_n):
    """(K, N) -> (K/16, N*16): every 16x16 tile flattened row-major, tiles of a tile-row side by side."""
    return q_w.reshape(size_k // 16, 16, size_n // 16, 16).permute(0, 2, 1, 3).reshape(size_k // 16, size_n * 16)


def marlin_qqq_pack(q_w, size_k, size_n, group_size):
    """Integer codes (K, N) -> int32 (K/16, N*16/8) in the reference's layout (marlin_utils.py:33-68)."""
    assert tuple(q_w.shape) == (size_k, size_n) and size_k % 16 == 0 and size_n % 64 == 0
    quant_type = "per-channel" if group_size in (-1, size_k) else "per-group"
    perm = marlin_qqq_weight_perm(quant_type)
    t = _tile_rows(q_w.to(torch.int64).cpu(), size_k, size_n)
    t = t.reshape(-1, perm.numel())[:, perm].reshape(t.shape) & 0xF
    shifts = (4 * torch.arange(8, dtype=torch.int64)).reshape(1, 1, 8)
    words = (t.reshape(t.shape[0], -1, 8) << shifts).sum(dim=2)
    return torch.from_numpy(words.numpy().astype(np.uint32).view(np.int32))


def marlin_qqq_unpack(packed, size_k, size_n, group_size):
    """Inverse of marlin_qqq_pack: int32 (K/16, N*2) -> int32 nibbles (K, N) in [0, 15]."""
    assert tuple(packed.shape) == (size_k // 16, size_n * 2)
    quant_type = "per-channel" if group_size in (-1, size_k) else "per-group"
    perm = marlin_qqq_weight_perm(quant_type)
    words = torch.from_numpy(packed.cpu().numpy().view(np.uint32).astype(np.int64))
    shifts = (4 * torch.arange(8, dtype=torch.int64)).reshape(1, 1, 8)
    t = ((words.unsqueeze(2) >> shifts) & 0xF).reshape(size_k // 16, size_n * 16)
    chunks = t.reshape(-1, perm.numel())
    out = torch.empty_like(chunks)
    out[:, perm] = chunks
    out = out.reshape(size_k // 16, size_n // 16, 16, 16).permute(0, 2, 1, 3).reshape(size_k, size_n)
    return out.to(torch.int32)


def marlin_qqq_permute_scales(s_group, s_channel, size_k, size_n, group_size):
    """Natural column order -> the reference's (marlin_utils.py:121-133)."""
    sp, sps = marlin_qqq_scale_perms()
    if group_size not in (-1, size_k):
        s_group = s_group.reshape(-1, sp.numel())[:, sp].reshape(-1, size_n).contiguous()
    s_channel = s_channel.reshape(-1, sps.numel())[:, sps].reshape(-1, size_n).contiguous()
    return s_group, s_channel


def marlin_qqq_unpermute_scales(s_group, s_channel, size_k, size_n, group_size):
    """The reference's column order -> natural."""
    sp, sps = marlin_qqq_scale_perms()
    if group_size not in (-1, size_k) and s_group.numel():
        g = s_group.reshape(-1, sp.numel())
        nat = torch.empty_like(g)
        nat[:, sp] = g
        s_group = nat.reshape(-1, size_n).contiguous()
    c = s_channel.reshape(-1, sps.numel())
    nat = torch.empty_like(c)
    nat[:, sps] = c
    return s_group, nat.reshape(-1, size_n).contiguous()


def marlin_qqq_to_native(weight, s_group, s_channel, size_k, size_n, group_size=128):
    """A reference W4A8 layer's buffers (``weight`` int32 (K/16, 2N), ``s_group`` fp16 (K/g, N) or empty,
    ``s_channel`` fp32 (1, N)) -> this library's (``weight`` uint8 (N, K/2), s_group, s_channel in natural
    column order).  The codes themselves are unchanged: offset-8 codes in the grouped scheme, two's
    complement nibbles in the per-channel scheme."""
    if s_group.numel() == 0:
        group_size = -1
    codes = marlin_qqq_unpack(weight, size_k, size_n, group_size)
    s_group, s_channel = marlin_qqq_unpermute_scales(s_group.cpu(), s_channel.cpu(), size_k, size_n, group_size)
    if s_group.numel() == 0:
        s_group = s_group.reshape(0, size_n)
    return pack_w4a8(codes), s_group, s_channel

"""Offline 4-bit weight quantisation for the W4A8 linears and this library's weight packing.

Numerics follow quamba/marlin_utils.py:139-262 (``get_w4a8_quantize_weights`` / ``w4a8_quantize``):
group scale = 2 * max|w_group| / 15, code = clamp(round(w / s) + 8, 0, 15), second-level int8
channel scale = max_k |w_ref| / 127, fused fp16 group scale = s_group / s_channel; per-channel
mode: code = clamp(round(w / (max|w| / 7)), -7, 7) as a signed nibble, s_channel /= 16.
Only the storage differs: codes are packed for the gfx950 kernel (``pack_w4a8``) and the scales are
kept in natural column order (the reference permutes both for its tensor-core tiles).
"""
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

"""Symmetric absmax quantisation helpers used by the modules' ``from_fp16`` constructors.

Semantics follow quamba/quant_utils.py:15-27 (per-tensor absmax, clamp of the maximum at 1e-5,
round-half-even via torch.round, values returned un-cast) and quamba/qSelectiveScan.py:12-18.
"""
import torch


def _quant_range(n_bits, sym=True):
    if sym:
        return -(2 ** (n_bits - 1)), 2 ** (n_bits - 1) - 1
    return 0, 2 ** n_bits - 1


@torch.no_grad()
def quantize_tensor_per_tensor_absmax(w, n_bits=8, clip_ratio=1.0):
    """Returns (rounded-and-clamped tensor in w's dtype, fp32 scale tensor)."""
    q_min, q_max = _quant_range(n_bits)
    w_max = w.abs().amax().clamp(min=1e-5)
    if clip_ratio < 1.0:
        w_max = w_max * clip_ratio
    scale = w_max / q_max
    q = torch.clamp(torch.round(w / scale), q_min, q_max)
    return q, scale.float()


@torch.no_grad()
def quantize_weight_per_tensor_absmax(w, n_bits=8):
    """Out-of-place variant of the helper the scan module uses for A_log / D / dt_bias."""
    q_max = 2 ** (n_bits - 1) - 1
    scale = w.abs().max().clamp(min=1e-5) / q_max
    return torch.round(w / scale), scale

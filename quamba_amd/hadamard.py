"""QHadamard: Hadamard rotation of the last dimension fused with int8 quantisation.

Drop-in for quamba/qHadamard.py:8-38 (module) and quamba/hadamard_utils.py:49-65 (choice of transform):
dim = 12 * 2^k uses the 12-point Paley matrix on the high index, dim = 40 * 2^k the 40-point one, any
other dim must be a power of two; the 1/sqrt(dim) normalisation and the output scale are folded into
the single multiplier the kernel applies before rounding.  ``x_H_scale`` travels through the state
dict as a Python float, as in the reference.
"""
import math

import torch

from . import ops


def _is_pow2(n):
    return n > 0 and (n & (n - 1)) == 0


def get_qhad_fn(dim):
    """(transform, N, had_scale) like quamba/hadamard_utils.py:49-65; the transform is the same function
    for every N here (the kernel picks the factorisation from dim)."""
    had_scale = 1.0 / math.sqrt(dim)
    if dim % 12 == 0:
        assert _is_pow2(dim // 12)
        N = 12
    elif dim % 40 == 0:
        assert _is_pow2(dim // 40)
        N = 40
    else:
        assert _is_pow2(dim)
        N = 2
    return ops.hadamard_quant, N, had_scale


class QHadamard(torch.nn.Module):

    def __init__(self, dim, x_H_scale=1.0):
        super().__init__()
        self.dim = dim
        self.x_H_scale = x_H_scale
        self.transform_fn, self.N, self.had_scale = get_qhad_fn(dim)
        self._register_state_dict_hook(self._store_scale)
        self._register_load_state_dict_pre_hook(self._load_scale)

    def _store_scale(self, module, state_dict, prefix, local_metadata):
        state_dict[prefix + "x_H_scale"] = self.x_H_scale
        return state_dict

    def _load_scale(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        self.x_H_scale = float(state_dict.pop(prefix + "x_H_scale"))

    @torch.no_grad()
    def forward(self, x):
        return self.transform_fn(x, self.had_scale / float(self.x_H_scale))

    def __repr__(self):
        return f"QHadamard(dim={self.dim})"

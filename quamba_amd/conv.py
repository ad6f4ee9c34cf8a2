"""QCausalConv1D: Mamba1 depthwise causal conv on int8 activations (int8 in, int8 out, fused SiLU).

Drop-in for quamba/qConvLayer.py:11-127: same constructor, buffers (``weight`` int8 (D,k),
``bias`` int8 (D)), Python-float scales carried through the state dict by hooks, ``from_fp16``,
``forward`` and ``update``.
"""
import torch
import torch.nn as nn

from . import ops
from .quant_utils import quantize_tensor_per_tensor_absmax

_SCALE_KEYS = ("weight_scale", "bias_scale", "input_scale", "output_scale")


class QCausalConv1D(nn.Module):

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1, groups=1,
                 bias=True, device=None, **kwargs):
        super().__init__()
        assert in_channels == out_channels == groups, "QCausalConv1D only supports in_channels == out_channels == groups"
        if isinstance(kernel_size, tuple):
            assert len(kernel_size) == 1, "QCausalConv1D only supports 1D kernel_size"
            kernel_size = kernel_size[0]
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.kernel_size = kernel_size
        self.stride = stride
        self.padding = padding
        self.dilation = dilation
        self.groups = groups
        self.register_buffer("weight", torch.empty((in_channels, kernel_size), dtype=torch.int8, device=device))
        if bias is not None and bias is not False:
            self.register_buffer("bias", torch.empty((in_channels,), dtype=torch.int8, device=device))
        else:
            self.bias = None
        self.weight_scale = 0.0
        self.bias_scale = 0.0
        self.input_scale = 0.0
        self.output_scale = 0.0
        self._register_state_dict_hook(self._store_scales)
        self._register_load_state_dict_pre_hook(self._load_scales)

    @classmethod
    def from_fp16(cls, originalLayer: nn.Conv1d, input_scale=1.0, output_scale=1.0):
        device = originalLayer.weight.device
        q = cls(originalLayer.in_channels, originalLayer.out_channels, originalLayer.kernel_size,
                originalLayer.stride, originalLayer.padding, originalLayer.dilation, originalLayer.groups,
                originalLayer.bias, device=device)
        q.input_scale = float(input_scale)
        q.output_scale = float(output_scale)
        w_q, w_s = quantize_tensor_per_tensor_absmax(originalLayer.weight.detach().clone(), n_bits=8)
        q.weight = w_q.to(torch.int8).reshape(w_q.shape[0], w_q.shape[-1]).contiguous().to(device)
        q.weight_scale = w_s.item()
        if originalLayer.bias is not None:
            b_q, b_s = quantize_tensor_per_tensor_absmax(originalLayer.bias.detach().clone(), n_bits=8)
            q.bias = b_q.to(torch.int8).contiguous().to(device)
            q.bias_scale = b_s.item()
        else:
            q.bias = None
            q.bias_scale = 1.0
        return q

    def _store_scales(self, module, state_dict, prefix, local_metadata):
        for k in _SCALE_KEYS:
            state_dict[prefix + k] = getattr(self, k)
        return state_dict

    def _load_scales(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        for k in _SCALE_KEYS:
            setattr(self, k, float(state_dict.pop(prefix + k)))

    @torch.no_grad()
    def forward(self, x):
        return ops.causal_conv1d_fwd(x, self.input_scale, self.weight, self.weight_scale, self.output_scale,
                                     self.bias_scale, self.bias, None, None, None, True)

    @torch.no_grad()
    def update(self, x, conv_state):
        """conv_state is shifted in place."""
        return ops.causal_conv1d_update(x, conv_state, self.input_scale, self.weight, self.weight_scale,
                                        self.output_scale, self.bias_scale, self.bias, True)

    def __repr__(self):
        return (f"QCausalConv1D({self.out_channels}, {self.in_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride})")

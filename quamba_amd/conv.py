"""QCausalConv1D: Mamba1 depthwise causal conv on int8 activations (int8 in, int8 out, fused SiLU).
Quamb2Conv1D: Mamba2 conv over the concatenated xBC channels with split scales and three outputs.

Drop-ins for quamba/qConvLayer.py:11-127 and :129-341: same constructors, buffers (``weight`` int8
(D,k), ``bias`` int8 (D), and for the Mamba2 conv ``x_head_group_range``, ``x_dim_group_range``,
``x_out_scales``, ``B_out_scales``, ``C_out_scales``), Python-float scales carried through the state
dict by hooks, ``from_fp16``, ``forward`` and ``update``.
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
    def forward(self, x, also_channel_last=False):
        """int8 (batch, dim, seqlen) -> int8, same strides.  ``also_channel_last=True`` returns the pair
        (out, out as a contiguous (batch, seqlen, dim) tensor), both written by the one kernel."""
        return ops.causal_conv1d_fwd(x, self.input_scale, self.weight, self.weight_scale, self.output_scale,
                                     self.bias_scale, self.bias, None, None, None, True,
                                     also_channel_last=also_channel_last)

    @torch.no_grad()
    def update(self, x, conv_state):
        """conv_state is shifted in place."""
        return ops.causal_conv1d_update(x, conv_state, self.input_scale, self.weight, self.weight_scale,
                                        self.output_scale, self.bias_scale, self.bias, True)

    def __repr__(self):
        return (f"QCausalConv1D({self.out_channels}, {self.in_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride})")


_SCALE_KEYS2 = ("x_scale", "B_scale", "C_scale", "wx_scale", "wB_scale", "wC_scale")
_BIAS_SCALE_KEYS2 = ("bx_scale", "bB_scale", "bC_scale")


class Quamb2Conv1D(nn.Module):
    """Mamba2 xBC conv (quamba/qConvLayer.py:129-341).  ``forward`` takes xBC int8 (batch, dim, seqlen) in
    channel-contiguous memory (a transposed view of in_proj's output) and returns int8 x, B, C."""

    def __init__(self, x_dim, x_headdim, d_state, n_groups, x_nhead_group, x_ndim_group, in_channels, out_channels,
                 kernel_size, stride=1, padding=0, dilation=1, groups=1, bias=True, device=None, **kwargs):
        super().__init__()
        self.x_dim = x_dim
        self.x_headdim = x_headdim
        self.d_state = d_state
        self.n_groups = n_groups
        self.x_nhead_group = x_nhead_group
        self.x_ndim_group = x_ndim_group
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
        self.x_scale = self.B_scale = self.C_scale = 0.0
        self.wx_scale = self.wB_scale = self.wC_scale = 0.0
        self.register_buffer("weight", torch.empty((in_channels, kernel_size), dtype=torch.int8, device=device))
        if bias is not None and bias is not False:
            self.register_buffer("bias", torch.empty((in_channels,), dtype=torch.int8, device=device))
            self.bx_scale = self.bB_scale = self.bC_scale = 0.0
        else:
            self.bias = None
            self.bx_scale = self.bB_scale = self.bC_scale = None
        self._register_state_dict_hook(self._store_scales)
        self._register_load_state_dict_pre_hook(self._load_scales)
        if x_nhead_group > 0 and x_ndim_group > 0:
            self.register_buffer("x_head_group_range", torch.empty((n_groups, x_nhead_group), dtype=torch.int32, device=device))
            self.register_buffer("x_dim_group_range",
                                 torch.empty((n_groups, x_nhead_group, x_ndim_group), dtype=torch.int32, device=device))
            self.register_buffer("x_out_scales",
                                 torch.empty((n_groups, x_nhead_group, x_ndim_group), dtype=torch.float32, device=device))
        elif x_nhead_group == 0 and x_ndim_group == 0:
            self.x_head_group_range = None
            self.x_dim_group_range = None
            self.register_buffer("x_out_scales", torch.empty((1,), dtype=torch.float32, device=device))
        else:
            raise ValueError("x_nhead_group and x_ndim_group must be both zero or both non-zero")
        self.register_buffer("B_out_scales", torch.empty((n_groups,), dtype=torch.float32, device=device))
        self.register_buffer("C_out_scales", torch.empty((n_groups,), dtype=torch.float32, device=device))

    @classmethod
    def from_fp16(cls, originalLayer: nn.Conv1d, x_dim, x_headdim, d_state, n_groups, x_scale, B_scale, C_scale,
                  x_out_scales, B_out_scales, C_out_scales, x_head_group_range, x_dim_group_range):
        if x_head_group_range is not None and x_dim_group_range is not None:
            assert x_head_group_range.dim() == 2, "x_head_group_range must have shape [n_ssd_group, x_nhead_group]"
            assert x_dim_group_range.dim() == 3, "x_dim_group_range must have shape [n_ssd_group, x_nhead_group, n_dim_group]"
            x_nhead_group, x_ndim_group = x_head_group_range.shape[1], x_dim_group_range.shape[2]
        elif x_head_group_range is None and x_dim_group_range is None:
            x_nhead_group = x_ndim_group = 0
        else:
            raise ValueError("x_head_group_range and x_dim_group_range must be both None or both not None")
        device = originalLayer.weight.device
        q = cls(x_dim, x_headdim, d_state, n_groups, x_nhead_group, x_ndim_group, originalLayer.in_channels,
                originalLayer.out_channels, originalLayer.kernel_size, originalLayer.stride, originalLayer.padding,
                originalLayer.dilation, originalLayer.groups, originalLayer.bias, device=device)
        q.x_scale, q.B_scale, q.C_scale = float(x_scale), float(B_scale), float(C_scale)
        q.x_head_group_range = x_head_group_range.to(device=device, dtype=torch.int32).contiguous() \
            if x_head_group_range is not None else None
        q.x_dim_group_range = x_dim_group_range.to(device=device, dtype=torch.int32).contiguous() \
            if x_dim_group_range is not None else None
        q.x_out_scales = x_out_scales.to(device=device, dtype=torch.float32).contiguous()
        q.B_out_scales = B_out_scales.to(device=device, dtype=torch.float32).contiguous()
        q.C_out_scales = C_out_scales.to(device=device, dtype=torch.float32).contiguous()
        parts = [x_dim, d_state * n_groups, d_state * n_groups]
        weight = originalLayer.weight.detach().clone().to(torch.float32)
        weight = weight.reshape(weight.shape[0], weight.shape[-1])
        w_q, w_s = [], []
        for w in torch.split(weight, parts, dim=0):
            wi, ws = quantize_tensor_per_tensor_absmax(w.contiguous(), n_bits=8, clip_ratio=1.0)
            w_q.append(wi.to(torch.int8))
            w_s.append(ws.item())
        q.weight = torch.cat(w_q, dim=0).contiguous().to(device)
        q.wx_scale, q.wB_scale, q.wC_scale = w_s
        if originalLayer.bias is not None:
            bias = originalLayer.bias.detach().clone().to(torch.float32)
            b_q, b_s = [], []
            for bpart in torch.split(bias, parts, dim=0):
                bi, bs = quantize_tensor_per_tensor_absmax(bpart.contiguous(), n_bits=8, clip_ratio=1.0)
                b_q.append(bi.to(torch.int8))
                b_s.append(bs.item())
            q.bias = torch.cat(b_q, dim=0).contiguous().to(device)
            q.bx_scale, q.bB_scale, q.bC_scale = b_s
        else:
            q.bias = None
            q.bx_scale = q.bB_scale = q.bC_scale = None
        return q

    def _store_scales(self, module, state_dict, prefix, local_metadata):
        for k in _SCALE_KEYS2:
            state_dict[prefix + k] = getattr(self, k)
        if self.bias is not None:
            for k in _BIAS_SCALE_KEYS2:
                state_dict[prefix + k] = getattr(self, k)
        return state_dict

    def _load_scales(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        for k in _SCALE_KEYS2:
            setattr(self, k, float(state_dict.pop(prefix + k)))
        if self.bias is not None:
            for k in _BIAS_SCALE_KEYS2:
                setattr(self, k, float(state_dict.pop(prefix + k)))

    def _args(self):
        return (self.x_scale, self.B_scale, self.C_scale, self.x_dim, self.x_headdim, self.d_state, self.n_groups,
                self.x_head_group_range, self.x_dim_group_range, self.x_out_scales, self.B_out_scales,
                self.C_out_scales, self.weight, self.wx_scale, self.wB_scale, self.wC_scale, self.bias,
                self.bx_scale, self.bB_scale, self.bC_scale, None, None, None, True)

    @torch.no_grad()
    def forward(self, xBC):
        return ops.quamba2_conv1d_fwd(xBC, *self._args())

    @torch.no_grad()
    def update(self, xBC, conv_state):
        """conv_state is shifted in place."""
        return ops.quamba2_conv1d_update(xBC, conv_state, *self._args())

    def __repr__(self):
        return (f"Quamb2Conv1D({self.out_channels}, {self.in_channels}, kernel_size={self.kernel_size}, "
                f"stride={self.stride})")

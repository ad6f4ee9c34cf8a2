"""W8A8 linear layers: int8 activations x int8 weights on the int8 matrix cores, scale epilogue.

Drop-ins for quamba/qLinearLayer.py:539-823 (W8A8B8O8Linear, W8A8B8O8LinearParallel,
W8A8B16O16Linear): same constructors, buffers (``weight`` int8 of shape (in, out+pad) with
strides (1, in), ``a``, ``b`` fp32) and state-dict keys, ``from_fp16``, ``forward`` and
``to_seqlen_last``.
"""
import torch
import torch.nn as nn

from . import ops
from .quant_utils import quantize_tensor_per_tensor_absmax


def _default_device():
    return torch.device("cuda")


class _W8A8Base(nn.Module):
    _b_per_channel = False

    def __init__(self, in_features, out_features, device=None):
        super().__init__()
        device = _default_device() if device is None else device
        self.bias = None
        self.in_features = in_features
        self.out_features = out_features
        self.pad_out = 0 if out_features % 16 == 0 else 16 - out_features % 16
        n = out_features + self.pad_out
        self.register_buffer("weight", torch.empty_strided((in_features, n), (1, in_features), dtype=torch.int8,
                                                           device=device))
        self.register_buffer("a", torch.empty((1, 1), dtype=torch.float32, device=device))
        self.register_buffer("b", torch.empty((1, n if self._b_per_channel else 1), dtype=torch.float32, device=device))

    def _quantized_weight(self, w_fp):
        q, s = quantize_tensor_per_tensor_absmax(w_fp, n_bits=8)
        return q, s

    def _set_weight(self, q_nk):
        """q_nk: (out, in) values; stored as the (in, out+pad) view with strides (1, in)."""
        if self.pad_out:
            q_nk = torch.nn.functional.pad(q_nk, (0, 0, 0, self.pad_out), "constant", 0)
        self.weight = q_nk.to(torch.int8).contiguous().t()

    def _mm(self, x2d, out_dtype):
        y = torch.empty((x2d.shape[0], self.out_features + self.pad_out), dtype=out_dtype, device=x2d.device)
        ops.scaled_mm_dq(y, x2d, self.weight, self.a, self.b)
        return y

    def _finish(self, y, x_shape):
        if self.pad_out:
            y = y[:, :-self.pad_out]
        return y.view(*x_shape[:-1], -1)


class _AlphaHooks:
    """``alpha`` (Python float used by the single-row path) travels through the state dict."""

    def _init_alpha(self):
        self.alpha = 0.0
        self._register_state_dict_hook(self._store_alpha)
        self._register_load_state_dict_pre_hook(self._load_alpha)

    def _store_alpha(self, module, state_dict, prefix, local_metadata):
        state_dict[prefix + "alpha"] = self.alpha
        return state_dict

    def _load_alpha(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        self.alpha = float(state_dict.pop(prefix + "alpha"))


class W8A8B8O8Linear(_W8A8Base, _AlphaHooks):
    """int8 in, int8 out; a = input_scale / output_scale, b = weight_scale (per tensor)."""

    def __init__(self, in_features, out_features, device=None):
        super().__init__(in_features, out_features, device)
        self._init_alpha()

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: float = 1.0, output_scale: float = 1.0):
        dev = originalLayer.weight.device
        q = cls(originalLayer.in_features, originalLayer.out_features, device=dev)
        w_q, w_s = q._quantized_weight(originalLayer.weight.detach())
        q._set_weight(w_q)
        q.a = torch.tensor([[input_scale / output_scale]], dtype=torch.float32, device=dev)
        q.b = torch.tensor([[w_s]], dtype=torch.float32, device=dev)
        q.alpha = (w_s * input_scale / output_scale).item()
        return q

    @torch.no_grad()
    def forward(self, x):
        x_shape = x.shape
        x2d = x.view(-1, x_shape[-1])
        if x2d.shape[0] == 1:
            y = torch.empty((1, self.out_features + self.pad_out), dtype=x.dtype, device=x.device)
            ops.scaled_mv_dq(y, self.weight.t(), x2d, self.alpha, 0.0)
        else:
            y = self._mm(x2d, x.dtype)
        return self._finish(y, x_shape)

    @torch.no_grad()
    def to_seqlen_last(self, x):
        """(B, L, in) -> (B, out, L) int8, computed as W x^T so that seqlen is the contiguous
        dimension; the result is a view with strides (L, B*L, 1) of a (out, B*L) buffer."""
        B, L, D = x.shape
        x2d = x.view(-1, D)
        pad_in = 0
        if x2d.shape[0] % 16 != 0:
            pad_in = 16 - x2d.shape[0] % 16
            x2d = nn.functional.pad(x2d, (0, 0, pad_in, 0), "constant", 0)
        y = torch.empty((self.out_features + self.pad_out, x2d.shape[0]), dtype=x.dtype, device=x.device)
        ops.scaled_mm_dq(y, self.weight.t(), x2d.t(), self.b, self.a)
        if self.pad_out:
            y = y[:-self.pad_out]
        if pad_in:
            y = y[:, pad_in:]
        return y.view(-1, B, L).transpose(0, 1)

    def __repr__(self):
        return f"W8A8B8O8Linear(in_features={self.in_features}, out_features={self.out_features})"


class W8A8B8O8LinearParallel(_W8A8Base):
    """int8 in, int8 out with one output scale per output segment: a = input_scale,
    b[n] = weight_scale(segment of n) / output_scale(segment of n)."""
    _b_per_channel = True

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: float, output_scales: list, out_split_dims: list):
        assert sum(out_split_dims) == originalLayer.out_features
        assert len(out_split_dims) == len(output_scales)
        dev = originalLayer.weight.device
        q = cls(originalLayer.in_features, originalLayer.out_features, device=dev)
        parts, scales, start = [], [], 0
        W = originalLayer.weight.detach()
        for dim, o_scale in zip(out_split_dims, output_scales):
            w_q, w_s = q._quantized_weight(W[start:start + dim])
            parts.append(w_q)
            scales.extend([w_s.item() / o_scale] * dim)
            start += dim
        scales.extend([0] * q.pad_out)
        q._set_weight(torch.cat(parts, dim=0))
        q.a = torch.tensor([[input_scale]], dtype=torch.float32, device=dev)
        q.b = torch.tensor([scales], dtype=torch.float32, device=dev)
        return q

    @torch.no_grad()
    def forward(self, x):
        x_shape = x.shape
        x2d = x.view(-1, x_shape[-1])
        if x2d.shape[0] == 1:
            y = torch.empty((1, self.out_features + self.pad_out), dtype=x.dtype, device=x.device)
            ops.w8a8o8_gemv(y, self.weight.t(), x2d, self.b, self.a)
        else:
            y = self._mm(x2d, x.dtype)
        return self._finish(y, x_shape)

    def __repr__(self):
        return f"W8A8B8O8LinearParallel(in_features={self.in_features}, out_features={self.out_features})"


class W8A8B16O16Linear(_W8A8Base, _AlphaHooks):
    """int8 in, fp16 out; a = input_scale, b = weight_scale."""

    def __init__(self, in_features, out_features, device=None):
        super().__init__(in_features, out_features, device)
        self._init_alpha()

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: float = 1.0):
        dev = originalLayer.weight.device
        q = cls(originalLayer.in_features, originalLayer.out_features, device=dev)
        w_q, w_s = q._quantized_weight(originalLayer.weight.detach())
        q._set_weight(w_q)
        q.a = torch.tensor([[input_scale]], dtype=torch.float32, device=dev)
        q.b = torch.tensor([[w_s]], dtype=torch.float32, device=dev)
        q.alpha = (w_s * input_scale).item()
        return q

    @torch.no_grad()
    def forward(self, x):
        x_shape = x.shape
        x2d = x.view(-1, x_shape[-1]).contiguous()
        if x2d.shape[0] == 1:
            y = torch.empty((1, self.out_features + self.pad_out), dtype=torch.float16, device=x.device)
            ops.scaled_mv_dq(y, self.weight.t(), x2d, self.alpha, 0.0)
        else:
            y = self._mm(x2d, torch.float16)
        return self._finish(y, x_shape)

    def __repr__(self):
        return f"W8A8B16O16Linear(in_features={self.in_features}, out_features={self.out_features})"


# ------------------------------------------------------------------------------------------------
# W4A8: int8 activations x 4-bit weights (group 128 fp16 scales over a per-channel int8 scale)
# Drop-ins for quamba/qLinearLayer.py:139-536.  Buffer names are the reference's (workspace, weight,
# input_scale, s_channel, s_group); ``weight`` holds this library's packing (uint8 (N, K/2), see
# w4a8_utils.pack_w4a8) and the scales are in natural column order, so a reference checkpoint needs
# re-packing before it can be loaded here.
# ------------------------------------------------------------------------------------------------
from .w4a8_utils import marlin_qqq_to_native, w4a8_quantize  # noqa: E402


class _W4A8Base(nn.Module):
    _out_dtype = torch.float16

    def __init__(self, in_features, out_features, group_size=128, device=None, **kwargs):
        super().__init__()
        device = _default_device() if device is None else device
        self.bias = None
        self.in_features = in_features
        self.out_features = out_features
        self.size_n, self.size_k = out_features, in_features
        self.pad_out = 0 if out_features % 64 == 0 else 64 - out_features % 64
        self.size_n += self.pad_out
        self.register_buffer("workspace", torch.zeros(1, dtype=torch.int32, device=device))
        self.register_buffer("weight", torch.empty((self.size_n, self.size_k // 2), dtype=torch.uint8, device=device))
        self.register_buffer("input_scale", torch.empty((), dtype=torch.float32, device=device))
        self.register_buffer("s_channel", torch.empty((1, self.size_n), dtype=torch.float32, device=device))
        n_groups = self.size_k // group_size if self.size_k > 128 else 0
        self.register_buffer("s_group", torch.empty((n_groups, self.size_n), dtype=torch.float16, device=device))

    @classmethod
    def _from_fp16(cls, originalLayer, input_scale, out_scales):
        assert input_scale.numel() == 1, "Only support per-tensor input scale"
        assert originalLayer.bias is None, "Not support bias yet"
        bits, group_scale = 4, None
        group_size = 128 if originalLayer.in_features > 128 else -1
        if getattr(originalLayer, "apply_gptq", False):
            bits, group_size = originalLayer.bits, originalLayer.group_size
            group_scale = originalLayer.group_scale.to(torch.float16).cpu()
        assert bits == 4, "Only support 4-bit quantization"
        if group_size not in (-1, 128):
            raise ValueError("Only groupsize -1 and 128 are supported.")
        device = originalLayer.weight.device
        q = cls(originalLayer.in_features, originalLayer.out_features, group_size=128, device=device)
        W = originalLayer.weight.detach()
        channel_scale = (W.abs().amax(dim=1, keepdim=True) / 127.0).reshape(1, -1).float().cpu()
        W_t = W.cpu().to(torch.float16).t().contiguous()
        w_ref, packed, s_group, s_channel = w4a8_quantize(W_t, bits, group_size, group_scale, channel_scale,
                                                          out_scales=out_scales, pad_out=q.pad_out)
        q.size_k, q.size_n = w_ref.shape
        q.weight = packed.to(device)
        q.input_scale = input_scale.detach().reshape(()).float().to(device)
        q.s_group = s_group.to(device)
        q.s_channel = s_channel.to(device)
        q.w_ref = w_ref          # dequantised (K, N) weights, kept for tests (not a buffer)
        return q

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        """Accepts a state dict written by the reference's module of the same name: an int32 ``weight`` is
        Marlin-QQQ storage (quamba/qLinearLayer.py:160-162) and is re-packed, with its scales, on the way in;
        the reference's lock ``workspace`` has no counterpart here."""
        wkey = prefix + "weight"
        if wkey in state_dict and state_dict[wkey].dtype == torch.int32:
            w = state_dict[wkey]
            size_k, size_n = w.shape[0] * 16, w.shape[1] // 2
            packed, s_group, s_channel = marlin_qqq_to_native(w, state_dict[prefix + "s_group"],
                                                              state_dict[prefix + "s_channel"], size_k, size_n)
            state_dict[wkey] = packed
            state_dict[prefix + "s_group"] = s_group
            state_dict[prefix + "s_channel"] = s_channel
            state_dict[prefix + "workspace"] = torch.zeros(1, dtype=torch.int32)
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)

    def _gemm(self, x2d, transpose):
        fn = ops.w4a8o8_gemm if self._out_dtype == torch.int8 else ops.w4a8o16_gemm
        return fn(x2d, self.weight, self.input_scale.reshape(1), self.s_channel, self.s_group, self.workspace,
                  x2d.shape[0], self.size_n, self.size_k, transpose)

    @torch.no_grad()
    def forward(self, x):
        x_shape = x.shape
        y = self._gemm(x.reshape(-1, x_shape[-1]).contiguous(), False)
        if self.pad_out:
            y = y[:, :-self.pad_out]
        return y.view(*x_shape[:-1], -1)

    @torch.no_grad()
    def to_seqlen_last(self, x):
        """(B, L, in) -> (B, out, L): a view with strides (L, B*L, 1) of an (out, B*L) buffer."""
        B, L, D = x.shape
        y = self._gemm(x.reshape(-1, D).contiguous(), True)
        if self.pad_out:
            y = y[:-self.pad_out]
        return y.view(-1, B, L).transpose(0, 1)

    def __repr__(self):
        return f"{type(self).__name__}(in_features={self.in_features}, out_features={self.out_features})"


class W4A8B16O16Linear(_W4A8Base):
    _out_dtype = torch.float16

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: torch.Tensor):
        return cls._from_fp16(originalLayer, input_scale, None)


class W4A8B8O8Linear(_W4A8Base):
    _out_dtype = torch.int8

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: torch.Tensor, output_scale: torch.Tensor):
        assert output_scale.numel() == 1, "Only support per-tensor output scale"
        return cls._from_fp16(originalLayer, input_scale, output_scale.reshape(1).cpu())


class W4A8B8O8LinearParallel(_W4A8Base):
    _out_dtype = torch.int8

    @classmethod
    def from_fp16(cls, originalLayer: nn.Linear, input_scale: torch.Tensor, output_scales, out_split_dims):
        assert sum(out_split_dims) == originalLayer.out_features
        assert len(out_split_dims) == len(output_scales)
        per_channel = torch.cat([torch.as_tensor(s, dtype=torch.float32).reshape(1).repeat(d)
                                 for d, s in zip(out_split_dims, output_scales)]).cpu()
        return cls._from_fp16(originalLayer, input_scale, per_channel)

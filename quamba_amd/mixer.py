"""W8A8QMamba: the quantized Mamba1 mixer assembled from this package's operators.

The call order, tensor layouts and state handling of quamba/qMambaLayer.py:757-1010 (``W8A8QMamba``):
in_proj (seqlen-last int8) -> x | z halves -> causal conv -> x_proj -> dt | B | C -> dt_proj (seqlen-last)
-> selective scan with z gate -> Hadamard + quantisation -> out_proj (fp16).  ``step`` is the one-token
form with the rolling conv state and the recurrent state updated in place.  This is the caller the
operators are built for; it owns no arithmetic of its own.

Two things the reference does with a copy are done in place here because the kernels take strides:
the conv and the scan read the x and z halves of in_proj's buffer directly, and B / C are passed to the
scan as transposed views only when that is free (they are tiny; a contiguous copy is made otherwise).
"""
import copy
import math

import torch
import torch.nn as nn
import torch.nn.functional as F

from .conv import QCausalConv1D
from .hadamard import QHadamard
from .linear import (W4A8B8O8Linear, W4A8B8O8LinearParallel, W4A8B16O16Linear, W8A8B8O8Linear, W8A8B8O8LinearParallel,
                     W8A8B16O16Linear)
from .sscan import QSScan


class W8A8QMamba(nn.Module):
    # the linear layers of this precision (W4A8QMamba overrides them); dt_proj is W8A8 in both
    _in_proj_cls, _x_proj_cls, _out_proj_cls = W8A8B8O8Linear, W8A8B8O8Linear, W8A8B16O16Linear

    def __init__(self, d_model, d_state=16, d_conv=4, expand=2, dt_rank="auto", conv_bias=True, bias=False,
                 use_had_transform=True, layer_idx=None, device=None, state_dtype=torch.int8, **kwargs):
        super().__init__()
        assert bias is False, "Only support bias=False for now"
        assert use_had_transform, "the mixer is built with the Hadamard + quantisation op in front of out_proj"
        device = torch.device("cuda") if device is None else device
        self.d_model = d_model
        self.d_state = d_state
        self.d_conv = d_conv
        self.expand = expand
        self.d_inner = int(expand * d_model)
        self.dt_rank = math.ceil(d_model / 16) if dt_rank == "auto" else dt_rank
        self.layer_idx = layer_idx
        self.state_dtype = state_dtype        # int8 (the reference) or fp32 recurrent state
        self.in_proj = self._in_proj_cls(d_model, self.d_inner * 2, device=device)
        self.conv1d = QCausalConv1D(self.d_inner, self.d_inner, d_conv, groups=self.d_inner, padding=d_conv - 1,
                                    bias=conv_bias, device=device)
        self.x_proj = self._x_proj_cls(self.d_inner, self.dt_rank + 2 * d_state, device=device)
        self.dt_proj = W8A8B8O8Linear(self.dt_rank, self.d_inner, device=device)
        self.selective_scan = QSScan(d_state, self.d_inner, delta_softplus=True, device=device)
        self.had = QHadamard(self.d_inner, x_H_scale=1.0)
        self.out_proj = self._out_proj_cls(self.d_inner, d_model, device=device)

    @classmethod
    def from_fp16(cls, originalLayer, act_scales, use_had_transform=True):
        """originalLayer: an fp16 Mamba mixer exposing in_proj, conv1d, x_proj, dt_proj (nn modules),
        dt_proj_bias, A_log, D and the size attributes; act_scales: the calibration dict of
        quamba/qMambaLayer.py:814-889 (same keys).  out_proj's weight must already carry the rotation."""
        dev = originalLayer.in_proj.weight.device
        q = cls(originalLayer.d_model, originalLayer.d_state, originalLayer.d_conv, originalLayer.expand,
                originalLayer.dt_rank, use_had_transform=use_had_transform, layer_idx=getattr(originalLayer, "layer_idx", None),
                device=dev)
        s = lambda k: float(torch.as_tensor(act_scales[k]).item())
        q.in_proj = cls._in_proj_cls.from_fp16(copy.deepcopy(originalLayer.in_proj), cls._scale(act_scales, "in_proj:input"),
                                               cls._scale(act_scales, "in_proj:output"))
        q.conv1d = QCausalConv1D.from_fp16(copy.deepcopy(originalLayer.conv1d), s("in_proj:output"), s("x_proj:input"))
        q.x_proj = cls._x_proj_cls.from_fp16(copy.deepcopy(originalLayer.x_proj), cls._scale(act_scales, "x_proj:input"),
                                             cls._scale(act_scales, "x_proj:output"))
        q.dt_proj = W8A8B8O8Linear.from_fp16(copy.deepcopy(originalLayer.dt_proj), s("x_proj:output"), s("dt_proj:output"))
        q.selective_scan = QSScan.from_fp16(
            originalLayer.d_state, originalLayer.d_inner, originalLayer.A_log.clone(), D=originalLayer.D.clone(),
            dt_bias=originalLayer.dt_proj_bias.clone(), delta_softplus=True,
            ssm_state_scale=act_scales["ssm_state_act:input"], u_scale=act_scales["x_proj:input"],
            dt_scale=act_scales["dt_proj:output"], B_scale=act_scales["x_proj:output"],
            C_scale=act_scales["x_proj:output"], z_scale=act_scales["in_proj:output"])
        q.had.x_H_scale = s("out_proj:input")
        q.out_proj = cls._out_proj_cls.from_fp16(copy.deepcopy(originalLayer.out_proj), cls._scale(act_scales, "out_proj:input"))
        return q

    @staticmethod
    def _scale(act_scales, key):
        """The form the linear classes of this precision take an activation scale in (a float here)."""
        return float(torch.as_tensor(act_scales[key]).item())

    @torch.no_grad()
    def forward(self, hidden_states, inference_params=None, conv_state=None, ssm_state=None):
        """hidden_states int8 (B, L, d_model) -> fp16 (B, L, d_model).  With conv_state / ssm_state (or an
        inference_params cache) the states after the last token are stored into them."""
        batch, seqlen, _ = hidden_states.shape
        if inference_params is not None:
            conv_state, ssm_state = self._get_states_from_cache(inference_params, batch)
            if inference_params.seqlen_offset > 0:
                out, _, _ = self.step(hidden_states, conv_state, ssm_state)
                return out
        xz = self.in_proj.to_seqlen_last(hidden_states)                 # (B, 2D, L), strides (L, B*L, 1)
        x, z = xz.chunk(2, dim=1)                                       # views
        if conv_state is not None:
            conv_state.copy_(F.pad(x, (conv_state.shape[-1] - x.shape[-1], 0)))
        # the conv writes its output in both layouts: (B, D, L) for the scan, (B, L, D) for x_proj
        fused = x.stride(2) == 1 and x.stride(1) % 16 == 0 and x.stride(0) % 16 == 0 and x.data_ptr() % 16 == 0
        if fused:
            x, x_rows = self.conv1d(x, also_channel_last=True)
        else:
            x = self.conv1d(x)                                          # same strides as its input
            x_rows = x.transpose(1, 2).contiguous()
        x_dbl = self.x_proj(x_rows)                                     # (B, L, dt_rank + 2N)
        dt, B, C = torch.split(x_dbl, [self.dt_rank, self.d_state, self.d_state], dim=-1)
        # (the GEMM reads a row-strided operand in place when rows and base are 16-byte aligned)
        if dt.stride(1) % 16 or dt.stride(0) != seqlen * dt.stride(1) or dt.data_ptr() % 16:
            dt = dt.contiguous()
        dt = self.dt_proj.to_seqlen_last(dt)                            # (B, D, L)
        B = B.transpose(1, 2).contiguous()                              # (B, N, L)
        C = C.transpose(1, 2).contiguous()
        want_state = ssm_state is not None
        y = self.selective_scan(x, dt, B, C, z=z, return_last_state=want_state,
                                state_dtype=ssm_state.dtype if want_state else torch.int8)
        if want_state:
            y, last_state = y
            ssm_state.copy_(last_state)
        return self.out_proj(self.had(y))                               # (B, L, d_model) fp16

    @torch.no_grad()
    def step(self, hidden_states, conv_state, ssm_state):
        assert hidden_states.shape[1] == 1, "Only support decoding with 1 token at a time for now"
        xz = self.in_proj(hidden_states.squeeze(1))                     # (B, 2D)
        x, z = xz.chunk(2, dim=-1)
        x = self.conv1d.update(x, conv_state)
        x_db = self.x_proj(x)
        dt, B, C = torch.split(x_db, [self.dt_rank, self.d_state, self.d_state], dim=-1)
        # the GEMM reads a row-strided operand in place when rows and base are 16-byte aligned
        if dt.stride(0) % 16 or dt.data_ptr() % 16:
            dt = dt.contiguous()
        dt = self.dt_proj(dt)
        y, ssm_state = self.selective_scan.update(ssm_state, x, dt, B, C, z=z)
        out = self.out_proj(self.had(y))
        return out.unsqueeze(1), conv_state, ssm_state

    def allocate_inference_cache(self, batch_size, max_seqlen=None, dtype=None, **kwargs):
        device = self.out_proj.weight.device
        conv_state = torch.zeros(batch_size, self.d_inner, self.d_conv, device=device, dtype=torch.int8)
        ssm_state = torch.zeros(batch_size, self.d_inner, self.d_state, device=device, dtype=self.state_dtype)
        return conv_state, ssm_state

    def _get_states_from_cache(self, inference_params, batch_size, initialize_states=False):
        assert self.layer_idx is not None
        cache = inference_params.key_value_memory_dict
        if self.layer_idx not in cache:
            cache[self.layer_idx] = self.allocate_inference_cache(batch_size)
        conv_state, ssm_state = cache[self.layer_idx]
        if initialize_states:
            conv_state.zero_()
            ssm_state.zero_()
        return conv_state, ssm_state


class W4A8QMamba(W8A8QMamba):
    """The W4A8 Mamba1 mixer of quamba/qMambaLayer.py:512-756: the same chain with 4-bit in_proj, x_proj and
    out_proj (group size 128); dt_proj stays W8A8 as there."""
    _in_proj_cls, _x_proj_cls, _out_proj_cls = W4A8B8O8Linear, W4A8B8O8Linear, W4A8B16O16Linear

    @staticmethod
    def _scale(act_scales, key):
        return torch.as_tensor(act_scales[key])


class W4A8QMamba2(nn.Module):
    """The quantized Mamba2 mixer of quamba/qMamba2.py:735-1068 (``W4A8QMamba2``) on this package's
    operators: in_proj (W4A8, int8 out with one output scale per z | x | B | C | dt segment) -> xBC conv
    (three int8 outputs) -> SSD chunk scan -> gated RMS norm (fp16) -> Hadamard + quantisation -> out_proj
    (W4A8, fp16).  ``step`` is the one-token form.  ``from_fp16`` is not provided: it needs the grouping
    tables produced by the reference's calibration pipeline; the sub-modules' own ``from_fp16`` exist."""

    _in_proj_cls, _out_proj_cls = W4A8B8O8LinearParallel, W4A8B16O16Linear      # W8A8QMamba2 overrides them

    def __init__(self, d_model, d_state=128, d_conv=4, expand=2, headdim=64, d_ssm=None, ngroups=1, D_has_hdim=False,
                 rmsnorm=True, norm_before_gate=False, dt_limit=(0.0, float("inf")), bias=False, conv_bias=True,
                 chunk_size=256, use_had_transform=True, layer_idx=None, device=None, state_dtype=torch.int8,
                 x_nhead_group=4, x_ndim_group=4, **kwargs):
        super().__init__()
        from .chunk_scan import Quamba2ChunkScan
        from .conv import Quamb2Conv1D
        from .norm import QRMSNormGated
        assert bias is False, "Only support bias=False for now"
        assert rmsnorm, "Only support Mamba2 block with rmsnorm"
        assert use_had_transform, "the mixer is built with the Hadamard + quantisation op in front of out_proj"
        device = torch.device("cuda") if device is None else device
        self.d_model, self.d_state, self.d_conv, self.expand = d_model, d_state, d_conv, expand
        self.d_inner = expand * d_model
        self.headdim = headdim
        self.d_ssm = self.d_inner if d_ssm is None else d_ssm
        assert self.d_ssm == self.d_inner, "the gated-MLP split (d_ssm < d_inner) is not part of this mixer"
        self.ngroups = ngroups
        self.nheads = self.d_ssm // headdim
        self.chunk_size = chunk_size
        self.layer_idx = layer_idx
        self.state_dtype = state_dtype
        d_in_proj = 2 * self.d_inner + 2 * ngroups * d_state + self.nheads      # order: z, x, B, C, dt
        self.in_proj = self._in_proj_cls(d_model, d_in_proj, device=device)
        conv_dim = self.d_ssm + 2 * ngroups * d_state
        self.conv1d = Quamb2Conv1D(self.d_ssm, headdim, d_state, ngroups, x_nhead_group, x_ndim_group, conv_dim, conv_dim,
                                   d_conv, groups=conv_dim, padding=d_conv - 1, bias=conv_bias, device=device)
        self.qchunk_scan = Quamba2ChunkScan(self.d_ssm, headdim, d_state, ngroups, D_has_hdim, chunk_size, x_nhead_group,
                                            x_ndim_group, delta_softplus=True, dt_limit=dt_limit, device=device)
        self.norm = QRMSNormGated(self.d_ssm, eps=1e-5, norm_before_gate=norm_before_gate, group_size=self.d_ssm // ngroups,
                                  use_float16_output=True, device=device)
        self.had = QHadamard(self.d_inner, x_H_scale=1.0)
        self.out_proj = self._out_proj_cls(self.d_inner, d_model, device=device)

    def _split(self, zxbcdt):
        return torch.split(zxbcdt, [self.d_ssm, self.d_ssm + 2 * self.ngroups * self.d_state, self.nheads], dim=-1)

    @torch.no_grad()
    def forward(self, u, conv_state=None, ssm_state=None):
        """u int8 (B, L, d_model) -> fp16 (B, L, d_model); conv_state / ssm_state receive the states after
        the last token when given."""
        batch, seqlen, _ = u.shape
        z, xBC, dt = self._split(self.in_proj(u))                   # views of (B, L, d_in_proj)
        if conv_state is not None:
            xBC_t = xBC.transpose(1, 2)
            conv_state.copy_(F.pad(xBC_t, (self.d_conv - xBC_t.shape[-1], 0)))
        x, B, C = self.conv1d(xBC.transpose(1, 2))                  # (B, ch, L) views of (B, L, ch) buffers
        x = x.transpose(1, 2).reshape(batch, seqlen, self.nheads, self.headdim)
        B = B.transpose(1, 2).reshape(batch, seqlen, self.ngroups, self.d_state)
        C = C.transpose(1, 2).reshape(batch, seqlen, self.ngroups, self.d_state)
        want_state = ssm_state is not None
        y = self.qchunk_scan(x, dt, B, C, z=None, return_final_states=want_state,
                             **({"state_dtype": ssm_state.dtype} if want_state else {}))
        if want_state:
            y, last_state = y
            ssm_state.copy_(last_state)
        return self.out_proj(self._norm_had(y.reshape(batch, seqlen, self.d_ssm), z))

    def _norm_had(self, y, z):
        """Gated norm, then the Hadamard transform + quantisation: one kernel where the shape allows."""
        if self.norm.fuses_with(self.had):
            return self.norm.forward_hadamard(y, z, self.had)
        return self.had(self.norm(y, z))

    @torch.no_grad()
    def step(self, hidden_states, conv_state, ssm_state):
        assert hidden_states.shape[1] == 1, "Only support decoding with 1 token at a time for now"
        z, xBC, dt = self._split(self.in_proj(hidden_states.squeeze(1)))
        x, B, C = self.conv1d.update(xBC, conv_state)
        y = self.qchunk_scan.update(ssm_state, x, dt, B, C, z=None)
        out = self.out_proj(self._norm_had(y.reshape(y.shape[0], self.d_ssm), z))
        return out.unsqueeze(1), conv_state, ssm_state

    def allocate_inference_cache(self, batch_size, max_seqlen=None, dtype=None, **kwargs):
        device = self.out_proj.weight.device
        conv_dim = self.conv1d.weight.shape[0]
        conv_state = torch.zeros(batch_size, self.d_conv, conv_dim, device=device, dtype=torch.int8).transpose(1, 2)
        ssm_state = torch.zeros(batch_size, self.nheads, self.headdim, self.d_state, device=device, dtype=self.state_dtype)
        return conv_state, ssm_state


class W8A8QMamba2(W4A8QMamba2):
    """The W8A8 Mamba2 mixer of quamba/qMamba2.py:1071-1400: the same chain with int8 weights in in_proj (one
    output scale per z | x | B | C | dt segment) and out_proj."""
    _in_proj_cls, _out_proj_cls = W8A8B8O8LinearParallel, W8A8B16O16Linear

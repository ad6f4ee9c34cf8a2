"""Quamba2ChunkScan: Mamba2 SSD chunk scan over int8 x / dt / B / C with per-tensor scales or the
head- and channel-grouped x scales of Quamba2.

Drop-in for quamba/qChunkScan.py:17-246: same constructor, buffers (dt_bias fp16, A_log int8,
A_log_scale, D, D_scale, dt_scale, z_scale, ssm_state_scale, x_scales, x_head_group_range,
x_dim_group_range, B_scale, C_scale), ``from_fp16``, ``forward`` and ``update``.  The reference
keeps the recurrent state in int8; ``state_dtype=torch.float32`` keeps it in fp32.
"""
import torch
import torch.nn as nn

from . import ops
from .quant_utils import quantize_tensor_per_tensor_absmax


class Quamba2ChunkScan(nn.Module):

    def __init__(self, d_ssm, headdim, d_state, ngroups, D_has_hdim, chunk_size, nhead_groups=0, ndim_groups=0,
                 delta_softplus=True, quant_dt=True, quant_B=True, quant_C=True, quant_z=False,
                 dt_limit=(0.0, float("inf")), device=None, **kwargs):
        super().__init__()
        device = torch.device("cuda") if device is None else device
        kw = dict(device=device)
        self.d_ssm, self.headdim, self.d_state, self.ngroups = d_ssm, headdim, d_state, ngroups
        self.D_has_hdim, self.chunk_size = D_has_hdim, chunk_size
        self.nhead_groups, self.ndim_groups = nhead_groups, ndim_groups
        self.delta_softplus, self.dt_limit = delta_softplus, dt_limit
        nheads = d_ssm // headdim
        self.register_buffer("dt_bias", torch.empty(nheads, dtype=torch.float16, **kw))
        self.register_buffer("A_log", torch.empty(nheads, dtype=torch.int8, **kw))
        self.register_buffer("A_log_scale", torch.empty([], dtype=torch.float32, **kw))
        self.register_buffer("D", torch.empty(d_ssm if D_has_hdim else nheads, dtype=torch.int8, **kw))
        self.register_buffer("D_scale", torch.empty([], dtype=torch.float32, **kw))
        for name, flag in (("dt", quant_dt), ("z", quant_z)):
            if flag:
                self.register_buffer(f"{name}_scale", torch.empty([], dtype=torch.float32, **kw))
            else:
                setattr(self, f"{name}_scale", None)
        if nhead_groups > 0 and ndim_groups > 0:
            self.register_buffer("ssm_state_scale", torch.empty([ngroups, nhead_groups, ndim_groups, d_state], dtype=torch.float32, **kw))
            self.register_buffer("x_scales", torch.empty([ngroups, nhead_groups, ndim_groups], dtype=torch.float32, **kw))
            self.register_buffer("x_head_group_range", torch.empty([ngroups, nhead_groups], dtype=torch.int32, **kw))
            self.register_buffer("x_dim_group_range", torch.empty([ngroups, nhead_groups, ndim_groups], dtype=torch.int32, **kw))
            bc_shape = [ngroups]
        elif nhead_groups == 0 and ndim_groups == 0:
            self.register_buffer("ssm_state_scale", torch.empty([1], dtype=torch.float32, **kw))
            self.register_buffer("x_scales", torch.empty([1], dtype=torch.float32, **kw))
            self.x_head_group_range = None
            self.x_dim_group_range = None
            bc_shape = [1]
        else:
            raise ValueError("nhead_groups and ndim_groups must be both 0 or both not 0")
        for name, flag in (("B", quant_B), ("C", quant_C)):
            if flag:
                self.register_buffer(f"{name}_scale", torch.empty(bc_shape, dtype=torch.float32, **kw))
            else:
                setattr(self, f"{name}_scale", None)

    @classmethod
    def from_fp16(cls, d_ssm, headdim, d_state, ngroups, x_scales, x_head_group_range, x_dim_group_range, A_log,
                  chunk_size, ssm_state_scale, D=None, D_has_hdim=False, dt_bias=None, delta_softplus=True,
                  dt_scale=None, B_scale=None, C_scale=None, z_scale=None, dt_limit=(0.0, float("inf"))):
        dev = A_log.device
        nhg = x_head_group_range.shape[1] if x_head_group_range is not None else 0
        ndg = x_dim_group_range.shape[2] if x_dim_group_range is not None else 0
        q = cls(d_ssm, headdim, d_state, ngroups, D_has_hdim, chunk_size, nhg, ndg, delta_softplus,
                dt_limit=dt_limit, device=dev)
        A_q, A_s = quantize_tensor_per_tensor_absmax(A_log.float(), n_bits=8)
        q.A_log = A_q.to(torch.int8)
        q.A_log_scale = A_s.float().to(dev)
        if x_head_group_range is not None:
            q.ssm_state_scale = cls.get_ssm_state_scales(ssm_state_scale, ngroups, nhg, ndg, d_state, dev)
        else:
            q.ssm_state_scale = torch.as_tensor(ssm_state_scale, dtype=torch.float32, device=dev).reshape(1)
        if D is not None:
            D_q, D_s = quantize_tensor_per_tensor_absmax(D.float(), n_bits=8)
            q.D = D_q.to(torch.int8)
            q.D_scale = D_s.float().to(dev)
        else:
            q.D = None
        q.dt_bias = dt_bias.to(torch.float16) if dt_bias is not None else None
        for name, s in (("dt_scale", dt_scale), ("B_scale", B_scale), ("C_scale", C_scale), ("z_scale", z_scale)):
            setattr(q, name, torch.as_tensor(s, dtype=torch.float32, device=dev) if s is not None else None)
        q.x_scales = torch.as_tensor(x_scales, dtype=torch.float32, device=dev)
        q.x_head_group_range = None if x_head_group_range is None else x_head_group_range.to(dev)
        q.x_dim_group_range = None if x_dim_group_range is None else x_dim_group_range.to(dev)
        return q

    @staticmethod
    def get_ssm_state_scales(scales, ngroups, n_head_groups, n_dim_groups, dstates, device):
        if isinstance(scales, list):
            out = torch.empty((ngroups, n_head_groups, n_dim_groups, dstates), device=device)
            for g in range(ngroups):
                for idx, (_h_size, _ch_size, ch_scales) in enumerate(scales[g]):
                    out[g, idx, :, :] = ch_scales.to(device)
            return out
        return scales.to(device)

    @torch.no_grad()
    def forward(self, x, dt, B, C, z=None, return_final_states=False, state_dtype=torch.int8):
        y, final_states = ops.ssd_chunk_scan_combined_fwd(
            x, self.x_scales, dt, self.dt_scale, self.A_log, self.A_log_scale, B, self.B_scale, C, self.C_scale,
            self.ssm_state_scale, self.chunk_size, q_D=self.D, D_scale=self.D_scale, q_z=z,
            z_scale=self.z_scale if z is not None else None, dt_bias=self.dt_bias, dt_softplus=self.delta_softplus,
            dt_limit=self.dt_limit, x_head_group_range=self.x_head_group_range,
            x_dim_group_range=self.x_dim_group_range, final_state_dtype=state_dtype)
        return (y, final_states) if return_final_states else y

    @torch.no_grad()
    def update(self, ssm_state, x, dt, B, C, z=None):
        """One token: x (batch, d_ssm), dt (batch, nheads), B, C (batch, ngroups*d_state); ssm_state
        (batch, nheads, headdim, d_state) int8 (or fp32) updated in place.  Returns y fp16 (batch, nheads, headdim)."""
        batch = x.shape[0]
        nheads = self.d_ssm // self.headdim
        dt3 = dt.unsqueeze(-1).expand(batch, nheads, self.headdim)
        A3 = self.A_log.view(nheads, 1, 1).expand(nheads, self.headdim, self.d_state)
        D2 = None
        if self.D is not None:
            D2 = self.D.view(nheads, self.headdim) if self.D_has_hdim else self.D.view(nheads, 1).expand(nheads, self.headdim)
        b2 = self.dt_bias.view(nheads, 1).expand(nheads, self.headdim) if self.dt_bias is not None else None
        return ops.sscan_update(
            ssm_state, x.view(batch, nheads, self.headdim), self.x_scales, dt3, self.dt_scale, A3, self.A_log_scale,
            self.ssm_state_scale, B.view(batch, self.ngroups, self.d_state), self.B_scale,
            C.view(batch, self.ngroups, self.d_state), self.C_scale, D2, self.D_scale if self.D is not None else None,
            z, self.z_scale if z is not None else None, b2, None, self.delta_softplus,
            x_head_group_range=self.x_head_group_range, x_dim_group_range=self.x_dim_group_range)

    def __repr__(self):
        return f"Quamba2ChunkScan(d_ssm={self.d_ssm}, headdim={self.headdim}, d_state={self.d_state}, chunk_size={self.chunk_size})"

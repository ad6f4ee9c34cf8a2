"""QSScan: Mamba1 selective scan on int8 u/dt/B/C/z with int8 A_log, D and dt_bias.

Drop-in for quamba/qSelectiveScan.py:70-203: same constructor, buffers and ``from_fp16``;
``forward`` returns fp16 (batch, seqlen, dim) and, on request, the last state; ``update`` advances
the recurrent state by one token in place.  The reference keeps the recurrent state in int8
(``ssm_state_scale``); passing ``state_dtype=torch.float32`` to ``forward`` or an fp32 ``ssm_state``
to ``update`` keeps it in fp32 instead.
"""
import torch
import torch.nn as nn

from . import ops
from .quant_utils import quantize_weight_per_tensor_absmax


def quant_selective_scan_fn(u, scale_u, delta, scale_delta, A, scale_A, B, scale_B, C, scale_C, ssm_state_scale,
                            D=None, scale_D=None, z=None, scale_z=None, delta_bias=None, scale_delta_bias=None,
                            delta_softplus=False, return_last_state=False, state_dtype=torch.int8):
    """Functional form (quamba/qSelectiveScan.py:51-66).  last_state has shape (batch, dim, dstate)."""
    if u.stride(-1) != 1:
        u = u.contiguous()
    if delta.stride(-1) != 1:
        delta = delta.contiguous()
    if B.stride(-1) != 1:
        B = B.contiguous()
    if C.stride(-1) != 1:
        C = C.contiguous()
    if z is not None and z.stride(-1) != 1:
        z = z.contiguous()
    if B.dim() == 3:
        B = B.unsqueeze(1)
    if C.dim() == 3:
        C = C.unsqueeze(1)
    out, x = ops.sscan_fwd(u, scale_u, delta, scale_delta, A, scale_A, B, scale_B, C, scale_C, ssm_state_scale,
                           D, scale_D, z, scale_z, delta_bias, scale_delta_bias, delta_softplus,
                           state_dtype=state_dtype)
    return (out, x[:, :, -1, :]) if return_last_state else out


class QSScan(nn.Module):

    def __init__(self, d_state, d_inner, delta_softplus=True, device=None):
        super().__init__()
        device = torch.device("cuda") if device is None else device
        self.delta_softplus = delta_softplus
        one = lambda: torch.tensor(1.0, device=device, dtype=torch.float32)
        self.register_buffer("dt_bias", torch.empty((d_inner,), device=device, dtype=torch.int8))
        self.register_buffer("dt_bias_scale", one())
        self.register_buffer("A_log", torch.empty((d_inner, d_state), device=device, dtype=torch.int8))
        self.register_buffer("A_scale", one())
        self.register_buffer("D", torch.empty((d_inner,), device=device, dtype=torch.int8))
        self.register_buffer("D_scale", one())
        for name in ("u_scale", "dt_scale", "B_scale", "C_scale", "z_scale", "ssm_state_scale"):
            self.register_buffer(name, one())

    @classmethod
    def from_fp16(cls, d_state, d_inner, A_log, D=None, dt_bias=None, delta_softplus=True, ssm_state_scale=1.0,
                  u_scale=1.0, dt_scale=1.0, B_scale=1.0, C_scale=1.0, z_scale=1.0):
        device = A_log.device
        q = cls(d_state, d_inner, device=device)

        def as_scale(s):
            return torch.as_tensor(s, dtype=torch.float32, device=device).reshape(())

        A_q, A_s = quantize_weight_per_tensor_absmax(A_log.float(), n_bits=8)
        q.A_log = A_q.to(torch.int8)
        q.A_scale = A_s.float()
        if D is not None:
            D_q, D_s = quantize_weight_per_tensor_absmax(D.float(), n_bits=8)
            q.D = D_q.to(torch.int8)
            q.D_scale = D_s.float()
        else:
            q.D = None
        if dt_bias is not None:
            b_q, b_s = quantize_weight_per_tensor_absmax(dt_bias.float(), n_bits=8)
            q.dt_bias = b_q.to(torch.int8)
            q.dt_bias_scale = b_s.float()
        else:
            q.dt_bias = None
            q.dt_bias_scale = torch.tensor(0.0, device=device)
        q.u_scale, q.dt_scale, q.B_scale = as_scale(u_scale), as_scale(dt_scale), as_scale(B_scale)
        q.C_scale, q.z_scale, q.ssm_state_scale = as_scale(C_scale), as_scale(z_scale), as_scale(ssm_state_scale)
        q.delta_softplus = delta_softplus
        return q

    @torch.no_grad()
    def forward(self, u, dt, B, C, z=None, return_last_state=False, state_dtype=torch.int8):
        return quant_selective_scan_fn(
            u, self.u_scale[None], dt, self.dt_scale[None], self.A_log, self.A_scale[None],
            B, self.B_scale[None], C, self.C_scale[None], ssm_state_scale=self.ssm_state_scale[None],
            D=self.D, scale_D=self.D_scale[None] if self.D is not None else None,
            z=z, scale_z=self.z_scale[None],
            delta_bias=self.dt_bias, scale_delta_bias=self.dt_bias_scale[None] if self.dt_bias is not None else None,
            delta_softplus=self.delta_softplus, return_last_state=return_last_state, state_dtype=state_dtype)

    @torch.no_grad()
    def update(self, ssm_state, u, dt, B, C, z=None):
        y = ops.sscan_update(
            ssm_state, u, self.u_scale[None], dt, self.dt_scale[None], self.A_log, self.A_scale[None],
            self.ssm_state_scale[None], B, self.B_scale[None], C, self.C_scale[None],
            self.D, self.D_scale[None] if self.D is not None else None,
            z, self.z_scale[None] if z is not None else None,
            self.dt_bias, self.dt_bias_scale[None] if self.dt_bias is not None else None,
            self.delta_softplus)
        return y, ssm_state

    def __repr__(self):
        return "QSScan()"

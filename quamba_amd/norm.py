"""QRMSNormGated: gated RMS norm between the Mamba2 SSD scan and out_proj, fp16 in, int8 or fp16 out.

Drop-in for quamba/qNorm.py:93-177: fp16 ``weight`` buffer, Python-float ``z_scale`` / ``output_scale``
carried through the state dict, ``from_fp16``, and ``forward(x, q_z)`` returning the int8 tensor (static
output scale), the pair (int8 tensor, per-token scales) (no output scale), or fp16.
"""
import torch

from . import ops


class QRMSNormGated(torch.nn.Module):

    def __init__(self, hidden_size, eps=1e-5, group_size=None, norm_before_gate=True, use_float16_output=False,
                 device=None, dtype=None):
        super().__init__()
        self.eps = eps
        self.register_buffer("weight", torch.empty(hidden_size, device=device, dtype=torch.float16))
        self.bias = None
        self.group_size = group_size
        self.norm_before_gate = norm_before_gate
        self.use_float16_output = use_float16_output
        self.z_scale = 0.0
        self.output_scale = 0.0
        self._register_state_dict_hook(self._store_scales)
        self._register_load_state_dict_pre_hook(self._load_scales)

    @classmethod
    def from_fp16(cls, originalLayer, z_scale=None, output_scale=None, use_float16_output=False):
        q = cls(originalLayer.weight.shape[0], originalLayer.eps, originalLayer.group_size,
                originalLayer.norm_before_gate, use_float16_output, originalLayer.weight.device)
        q.weight = originalLayer.weight.detach().clone().to(torch.float16)
        if z_scale is not None:
            assert type(z_scale) is float, "Only support per-tensor static quant for input z"
            q.z_scale = z_scale
        if output_scale is not None:
            assert type(output_scale) is float, "Only support per-tensor static quant for output"
            q.output_scale = output_scale
        else:
            q.output_scale = None           # dynamic per-token scales are returned with the output
        return q

    def _store_scales(self, module, state_dict, prefix, local_metadata):
        state_dict[prefix + "z_scale"] = self.z_scale
        state_dict[prefix + "output_scale"] = self.output_scale
        return state_dict

    def _load_scales(self, state_dict, prefix, local_metadata, strict, missing_keys, unexpected_keys, error_msgs):
        self.z_scale = state_dict.pop(prefix + "z_scale")
        self.output_scale = state_dict.pop(prefix + "output_scale")

    @torch.no_grad()
    def forward(self, x, q_z=None):
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        if q_z is not None:
            assert q_z.shape == shape
            q_z = q_z.reshape(-1, shape[-1])
            if q_z.stride(-1) != 1:
                q_z = q_z.contiguous()
        y, scales = ops.qlayer_normgated_fwd(x2, self.weight, self.bias, self.eps, q_z=q_z, z_scale=self.z_scale,
                                             static_out_scale=self.output_scale, use_float16_output=self.use_float16_output,
                                             group_size=self.group_size, norm_before_gate=self.norm_before_gate,
                                             is_rms_norm=True)
        if self.use_float16_output or self.output_scale is not None:
            return y.reshape(shape)
        # one scale per (group, row); with a single group this is the reference's per-token shape
        ngroups = 1 if self.group_size is None else shape[-1] // self.group_size
        return y.reshape(shape), scales.reshape(shape[:-1]) if ngroups == 1 else scales.reshape(ngroups, *shape[:-1])

    def fuses_with(self, had):
        """True when ``had(self(x, q_z))`` can run as one kernel: fp16 output feeding a power-of-two transform
        of a shape the fused kernel covers."""
        dim = self.weight.shape[0]
        group = dim if self.group_size is None else self.group_size
        return self.use_float16_output and had.dim == dim and ops.normgated_hadamard_supported(dim, group)

    @torch.no_grad()
    def forward_hadamard(self, x, q_z, had):
        """``had(self(x, q_z))`` bit for bit, in one kernel (``had`` a QHadamard of the same width)."""
        assert self.fuses_with(had)
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        if q_z is not None:
            assert q_z.shape == shape
            q_z = q_z.reshape(-1, shape[-1])
            if q_z.stride(-1) != 1:
                q_z = q_z.contiguous()
        out = ops.qlayer_normgated_hadamard_quant(x2, self.weight, self.eps, had.had_scale / float(had.x_H_scale), q_z=q_z,
                                                  z_scale=self.z_scale, group_size=self.group_size,
                                                  norm_before_gate=self.norm_before_gate)
        return out.reshape(shape)

    def __repr__(self):
        return (f"QRMSNormGated(dim={self.weight.shape[0]}, eps={self.eps}, z_scale={self.z_scale}, "
                f"output_scale={self.output_scale}, use_float16_output={self.use_float16_output})")

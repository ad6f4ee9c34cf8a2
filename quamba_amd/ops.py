"""Functional operator layer: one Python function per extension entry point of the reference,
with the reference's argument order and error behaviour, each forwarding to the C ABI of
libquamba_amd.so on the tensor's device and torch's current stream.

Reference interfaces mirrored here:
  quant_causal_conv1d_cuda.fwd / .update   csrc/causal_conv1d/quant_causal_conv1d.cpp:76-226
  quant_sscan_cuda.fwd                     csrc/selective_scan/quant_sscan.cpp:122-265
  quant_sscan_update_triton                quamba/triton/selective_state_update.py:129-227
  quant_linear_cuda.cutlass_scaled_mm_dq   csrc/linear/quant_linear_fwd_kernel.cuh:356-378
"""
import ctypes as ct

import torch

from . import _lib
from ._lib import ptr


def _require(cond, msg):
    if not cond:
        raise RuntimeError(msg)


def _require_gpu(t, name):
    _require(t.is_cuda, f"{name} must be a GPU tensor (quamba_amd has no CPU path)")


# ----------------------------------------------------------------------------------------------
# causal conv1d
# ----------------------------------------------------------------------------------------------
def causal_conv1d_fwd(x, scale_x, weight, scale_w, scale_out, scale_b, bias=None, seq_idx=None,
                      initial_states=None, final_states_out=None, silu_activation=True, also_channel_last=False):
    """int8 (batch, dim, seqlen) -> int8 of the same shape and strides.  With ``also_channel_last`` the kernel
    writes the result a second time as a contiguous (batch, seqlen, dim) tensor (what x_proj reads; the
    reference's caller makes that copy in a separate pass, quamba/qMambaLayer.py:923) and both are returned."""
    _require(x.dtype == torch.int8 and weight.dtype == torch.int8, "x and weight must be int8")
    _require_gpu(x, "x")
    _require_gpu(weight, "weight")
    _require(x.dim() == 3, "x must have shape (batch, dim, seqlen)")
    batch, dim, seqlen = x.shape
    width = weight.shape[-1]
    _require(tuple(weight.shape) == (dim, width), "weight must have shape (dim, width)")
    _require(x.stride(2) == 1 or x.stride(1) == 1, "x must be contiguous along seqlen or along channels")
    _require(2 <= width <= 4, "causal_conv1d only supports width between 2 and 4")
    if bias is not None:
        _require(bias.dtype == torch.int8 and bias.is_cuda and tuple(bias.shape) == (dim,) and bias.stride(-1) == 1,
                 "bias must be a contiguous int8 GPU tensor of shape (dim,)")
    if seq_idx is not None:
        raise NotImplementedError("No implementation for seq_idx")
    if initial_states is not None:
        raise NotImplementedError("No implementation for initial_states")
    if final_states_out is not None:
        raise NotImplementedError("No implementation for final_states_out")
    out = torch.empty_like(x)  # preserves strides for dense (possibly permuted) inputs
    if out.stride() != x.stride():
        out = torch.empty_strided(x.shape, x.stride(), dtype=x.dtype, device=x.device)
    p = _lib.QaConvParams()
    p.batch, p.dim, p.seqlen, p.width = batch, dim, seqlen, width
    p.silu_activation = int(bool(silu_activation))
    p.x_batch_stride, p.x_c_stride, p.x_l_stride = x.stride()
    p.out_batch_stride, p.out_c_stride, p.out_l_stride = out.stride()
    p.weight_c_stride, p.weight_width_stride = weight.stride()
    p.x, p.weight, p.bias, p.out = ptr(x), ptr(weight), ptr(bias), ptr(out)
    p.scale_x, p.scale_w, p.scale_b, p.scale_out = float(scale_x), float(scale_w), float(scale_b), float(scale_out)
    out_t = None
    if also_channel_last:
        _require(x.numel() == 0 or (x.stride(2) == 1 and x.stride(1) % 16 == 0 and x.stride(0) % 16 == 0 and x.data_ptr() % 16 == 0),
                 "also_channel_last needs a seqlen-contiguous input with 16-byte aligned rows")
        out_t = torch.empty((batch, seqlen, dim), dtype=torch.int8, device=x.device)
        p.out_t = ptr(out_t)
        p.out_t_batch_stride, p.out_t_l_stride = out_t.stride(0), out_t.stride(1)
    with torch.cuda.device(x.device):
        st = _lib.lib().qa_causal_conv1d_fwd(ct.byref(p), _lib.current_stream(x.device))
    _lib.check(st, "causal_conv1d_fwd")
    return (out, out_t) if also_channel_last else out


def _conv_update_params(x, conv_state, scale_x, weight, scale_w, scale_out, scale_b, bias, silu_activation):
    """QaConvParams of one decode step and the output tensor they point at."""
    _require(x.dtype == torch.int8 and weight.dtype == torch.int8 and conv_state.dtype == torch.int8,
             "x, weight and conv_state must be int8")
    for t, n in ((x, "x"), (conv_state, "conv_state"), (weight, "weight")):
        _require_gpu(t, n)
    _require(x.dim() == 2, "x must have shape (batch, dim)")
    batch, dim = x.shape
    width = weight.shape[-1]
    _require(tuple(weight.shape) == (dim, width), "weight must have shape (dim, width)")
    _require(2 <= width <= 4, "causal_conv1d only supports width between 2 and 4")
    _require(conv_state.dim() == 3 and tuple(conv_state.shape[:2]) == (batch, dim)
             and conv_state.shape[2] in (width, width - 1),
             "conv_state must have shape (batch, dim, width) or (batch, dim, width-1)")
    if bias is not None:
        _require(bias.dtype == torch.int8 and bias.is_cuda and tuple(bias.shape) == (dim,) and bias.stride(-1) == 1,
                 "bias must be a contiguous int8 GPU tensor of shape (dim,)")
    out = torch.empty_like(x)
    p = _lib.QaConvParams()
    p.batch, p.dim, p.seqlen, p.width = batch, dim, 1, width
    p.silu_activation = int(bool(silu_activation))
    p.x_batch_stride, p.x_c_stride, p.x_l_stride = x.stride(0), x.stride(1), 1
    p.out_batch_stride, p.out_c_stride, p.out_l_stride = out.stride(0), out.stride(1), 1
    p.weight_c_stride, p.weight_width_stride = weight.stride()
    p.conv_state_batch_stride, p.conv_state_c_stride, p.conv_state_l_stride = conv_state.stride()
    p.conv_state_len = conv_state.shape[2]
    p.x, p.weight, p.bias, p.out, p.conv_state = ptr(x), ptr(weight), ptr(bias), ptr(out), ptr(conv_state)
    p.scale_x, p.scale_w, p.scale_b, p.scale_out = float(scale_x), float(scale_w), float(scale_b), float(scale_out)
    return p, out


def causal_conv1d_update(x, conv_state, scale_x, weight, scale_w, scale_out, scale_b, bias=None,
                         silu_activation=True):
    """One decode step: x int8 (batch, dim); conv_state int8 (batch, dim, width) or
    (batch, dim, width-1), shifted in place."""
    p, out = _conv_update_params(x, conv_state, scale_x, weight, scale_w, scale_out, scale_b, bias, silu_activation)
    with torch.cuda.device(x.device):
        st = _lib.lib().qa_causal_conv1d_update(ct.byref(p), _lib.current_stream(x.device))
    _lib.check(st, "causal_conv1d_update")
    return out


def mamba1_decode_step(x, conv_state, scale_x, weight, scale_w, scale_out, scale_b, bias, silu_activation,
                       state, q_dt, dt_scale, q_A_log, A_log_scale, ssm_state_scale, q_B, B_scale, q_C, C_scale,
                       q_D=None, D_scale=None, q_z=None, z_scale=None, dt_bias=None, dt_bias_scale=None,
                       dt_softplus=False, x_scale=None):
    """causal_conv1d_update followed by sscan_update on the conv's output, in one launch (qa_mamba1_decode_step):
    for decode loops whose dt, B and C are given, i.e. do not come from a projection of this step's conv output.
    Arguments as for the two calls; the scan's x scale is the conv's ``scale_out``: pass it again as ``x_scale``, a
    one-element fp32 GPU tensor, to keep the call free of host-to-device copies (graph capture).  conv_state and
    state are updated in place.  Returns (conv output int8, y fp16)."""
    pc, xc = _conv_update_params(x, conv_state, scale_x, weight, scale_w, scale_out, scale_b, bias, silu_activation)
    if x_scale is None:
        x_scale = torch.tensor([float(scale_out)], dtype=torch.float32, device=x.device)
    y = sscan_update(state, xc, x_scale, q_dt, dt_scale, q_A_log, A_log_scale, ssm_state_scale, q_B, B_scale, q_C,
                     C_scale, q_D, D_scale, q_z, z_scale, dt_bias, dt_bias_scale, dt_softplus, _conv_step=pc)
    return xc, y


# ----------------------------------------------------------------------------------------------
# Mamba1 selective scan
# ----------------------------------------------------------------------------------------------
def _scale1(t, name):
    _require(t is not None and t.dtype == torch.float32 and t.is_cuda and t.numel() == 1,
             f"{name} must be a one-element fp32 GPU tensor")
    return t


def _conv2_params(xBC, x_dim, x_headdim, d_state, n_groups, x_head_group_range, x_dim_group_range, x_scales,
                  scale_B_out, scale_C_out, weight, bias, dim):
    """Argument checks shared by the Mamba2 xBC conv entry points (conditions of
    csrc/causal_conv1d/quamba2_conv1d.cpp:125-186)."""
    _require(xBC.dtype == torch.int8 and weight.dtype == torch.int8, "xBC and weight must be int8")
    _require_gpu(xBC, "xBC")
    _require_gpu(weight, "weight")
    width = weight.shape[-1]
    _require(tuple(weight.shape) == (dim, width), "weight must have shape (dim, width)")
    if bias is not None:
        _require(bias.dtype == torch.int8 and bias.is_cuda and tuple(bias.shape) == (dim,) and bias.stride(-1) == 1,
                 "bias must be a contiguous int8 GPU tensor of shape (dim,)")
    _require(x_dim <= dim, "x_dim must less or equal to input dim")
    _require(x_dim % x_headdim == 0, "x_dim must be divided by x_headdim")
    _require(x_dim + 2 * d_state * n_groups == dim, "x_dim + 2*d_state*n_groups must be equal to total dim")
    p = _lib.QaConv2Params()
    p.dim, p.width = dim, width
    p.x_dim, p.x_headdim, p.d_state, p.n_groups = x_dim, x_headdim, d_state, n_groups
    for t, n in ((x_scales, "x_scales"), (scale_B_out, "scale_B_out"), (scale_C_out, "scale_C_out")):
        _require(t.dtype == torch.float32 and t.is_cuda and t.is_contiguous(), f"{n} must be a contiguous fp32 GPU tensor")
    if x_head_group_range is not None and x_dim_group_range is not None:
        for t in (x_head_group_range, x_dim_group_range):
            _require(t.dtype == torch.int32 and t.is_cuda and t.is_contiguous(), "group ranges must be contiguous int32 GPU tensors")
        _require(x_head_group_range.dim() == 2 and x_head_group_range.shape[0] == n_groups,
                 "x_head_group_range.shape[0] must be equal to total number of groups")
        _require(x_dim_group_range.dim() == 3 and x_dim_group_range.shape[0] == n_groups,
                 "x_dim_group_range.shape[0] must be equal to total number of groups")
        p.nhead_groups, p.ndim_groups = x_head_group_range.shape[1], x_dim_group_range.shape[2]
        _require(x_dim_group_range.shape[1] == p.nhead_groups,
                 "x_dim_group_range.shape[1] must be equal to total number of head groups")
        _require(x_scales.numel() == n_groups * p.nhead_groups * p.ndim_groups,
                 "number of x scales must be equal to total number of groups")
        _require(scale_B_out.numel() == n_groups and scale_C_out.numel() == n_groups,
                 "number of B / C scales must be equal to total number of SSD groups")
        p.x_head_group_range, p.x_dim_group_range = ptr(x_head_group_range), ptr(x_dim_group_range)
    else:
        _require(x_head_group_range is None and x_dim_group_range is None,
                 "x_head_group_range and x_dim_group_range must be both None or both not None")
        _require(x_scales.numel() == 1 and scale_B_out.numel() == 1 and scale_C_out.numel() == 1,
                 "number of x / B / C scales must be equal to 1")
    p.x_out_scales, p.B_out_scales, p.C_out_scales = ptr(x_scales), ptr(scale_B_out), ptr(scale_C_out)
    p.weight_c_stride, p.weight_width_stride = weight.stride()
    p.weight, p.bias = ptr(weight), ptr(bias)
    return p


def quamba2_conv1d_fwd(xBC, scale_x, scale_B, scale_C, x_dim, x_headdim, d_state, n_groups, x_head_group_range,
                       x_dim_group_range, x_scales, scale_B_out, scale_C_out, weight, scale_wx, scale_wB, scale_wC,
                       bias=None, scale_bx=None, scale_bB=None, scale_bC=None, seq_idx=None, initial_states=None,
                       final_states_out=None, silu_activation=True):
    """Mamba2 xBC conv forward (quamba2_conv1d_cuda.fwd, csrc/causal_conv1d/quamba2_conv1d.cpp:109-251).
    xBC int8 (batch, dim, seqlen) in channel-contiguous memory.  Returns x (batch, x_dim, seqlen), B and C
    (batch, n_groups*d_state, seqlen), int8, each a transposed view of a (batch, seqlen, channels) buffer."""
    _require(xBC.dim() == 3, "xBC must have shape (batch, dim, seqlen)")
    batch, dim, seqlen = xBC.shape
    _require(xBC.stride(1) == 1 and (xBC.stride(2) > 1 or dim == 1 or seqlen == 1), "only support channel_last")
    if seq_idx is not None:
        raise NotImplementedError("No implementation for seq_idx")
    if initial_states is not None:
        raise NotImplementedError("No implementation for initial_states")
    if final_states_out is not None:
        raise NotImplementedError("No implementation for final_states_out")
    p = _conv2_params(xBC, x_dim, x_headdim, d_state, n_groups, x_head_group_range, x_dim_group_range, x_scales,
                      scale_B_out, scale_C_out, weight, bias, dim)
    _require(2 <= p.width <= 4, "causal_conv1d only supports width between 2 and 4")
    bc = d_state * n_groups
    x = torch.empty((batch, seqlen, x_dim), dtype=torch.int8, device=xBC.device).transpose(1, 2)
    B = torch.empty((batch, seqlen, bc), dtype=torch.int8, device=xBC.device).transpose(1, 2)
    C = torch.empty((batch, seqlen, bc), dtype=torch.int8, device=xBC.device).transpose(1, 2)
    p.batch, p.seqlen = batch, seqlen
    p.silu_activation = int(bool(silu_activation))
    p.xBC_batch_stride, p.xBC_c_stride, p.xBC_l_stride = xBC.stride()
    p.x_batch_stride, p.x_c_stride, p.x_l_stride = x.stride()
    p.B_batch_stride, p.B_c_stride, p.B_l_stride = B.stride()
    p.C_batch_stride, p.C_c_stride, p.C_l_stride = C.stride()
    p.xBC, p.x, p.B, p.C = ptr(xBC), ptr(x), ptr(B), ptr(C)
    p.scale_x, p.scale_B, p.scale_C = float(scale_x), float(scale_B), float(scale_C)
    p.scale_wx, p.scale_wB, p.scale_wC = float(scale_wx), float(scale_wB), float(scale_wC)
    p.scale_bx, p.scale_bB, p.scale_bC = (float(v) if v is not None else 0.0 for v in (scale_bx, scale_bB, scale_bC))
    with torch.cuda.device(xBC.device):
        st = _lib.lib().qa_quamba2_conv1d_fwd(ct.byref(p), _lib.current_stream(xBC.device))
    _lib.check(st, "quamba2_conv1d_fwd")
    return x, B, C


def quamba2_conv1d_update(xBC, conv_state, scale_x, scale_B, scale_C, x_dim, x_headdim, d_state, n_groups,
                          x_head_group_range, x_dim_group_range, x_scales, scale_B_out, scale_C_out, weight,
                          scale_wx, scale_wB, scale_wC, bias=None, scale_bx=None, scale_bB=None, scale_bC=None,
                          seq_idx=None, initial_states=None, final_states_out=None, silu_activation=True):
    """One decode step of the Mamba2 xBC conv (quamba2_conv1d_cuda.update, quamba2_conv1d.cpp:254-379).
    xBC int8 (batch, dim); conv_state int8 (batch, dim, width) (or width-1), shifted in place.
    Returns x (batch, x_dim), B, C (batch, n_groups*d_state), int8."""
    _require(xBC.dim() == 2, "xBC must have shape (batch, dim)")
    batch, dim = xBC.shape
    p = _conv2_params(xBC, x_dim, x_headdim, d_state, n_groups, x_head_group_range, x_dim_group_range, x_scales,
                      scale_B_out, scale_C_out, weight, bias, dim)
    _require(2 <= p.width <= 4, "causal_conv1d only supports width between 2 and 4")
    _require(conv_state.dtype == torch.int8 and conv_state.is_cuda, "conv_state must be an int8 GPU tensor")
    _require(conv_state.dim() == 3 and tuple(conv_state.shape[:2]) == (batch, dim)
             and conv_state.shape[2] in (p.width, p.width - 1),
             "conv_state must have shape (batch, dim, width) or (batch, dim, width-1)")
    bc = d_state * n_groups
    x = torch.empty((batch, x_dim), dtype=torch.int8, device=xBC.device)
    B = torch.empty((batch, bc), dtype=torch.int8, device=xBC.device)
    C = torch.empty((batch, bc), dtype=torch.int8, device=xBC.device)
    p.batch, p.seqlen = batch, 1
    p.silu_activation = int(bool(silu_activation))
    p.xBC_batch_stride, p.xBC_c_stride = xBC.stride()
    p.x_batch_stride, p.x_c_stride = x.stride()
    p.B_batch_stride, p.B_c_stride = B.stride()
    p.C_batch_stride, p.C_c_stride = C.stride()
    p.conv_state_batch_stride, p.conv_state_c_stride, p.conv_state_l_stride = conv_state.stride()
    p.conv_state_len = conv_state.shape[2]
    p.xBC, p.x, p.B, p.C, p.conv_state = ptr(xBC), ptr(x), ptr(B), ptr(C), ptr(conv_state)
    p.scale_x, p.scale_B, p.scale_C = float(scale_x), float(scale_B), float(scale_C)
    p.scale_wx, p.scale_wB, p.scale_wC = float(scale_wx), float(scale_wB), float(scale_wC)
    p.scale_bx, p.scale_bB, p.scale_bC = (float(v) if v is not None else 0.0 for v in (scale_bx, scale_bB, scale_bC))
    with torch.cuda.device(xBC.device):
        st = _lib.lib().qa_quamba2_conv1d_update(ct.byref(p), _lib.current_stream(xBC.device))
    _lib.check(st, "quamba2_conv1d_update")
    return x, B, C


def hadamard_quant(x, scale):
    """int8 of round(H x * scale) along the last dimension (quant_hadamard.fast_hadamard_transform[_12N|_40N],
    csrc/hadamard/quant_hadamard.cpp).  x fp16 or fp32 (..., dim), dim = S * 2^k with S in {1, 12, 40}."""
    _require(x.dtype in (torch.float16, torch.float32), "x must be fp16 or fp32")
    _require_gpu(x, "x")
    shape = x.shape
    dim = shape[-1]
    x2 = x.reshape(-1, dim)
    if x2.stride(-1) != 1:
        x2 = x2.contiguous()
    out = torch.empty(x2.shape, dtype=torch.int8, device=x.device)
    p = _lib.QaHadamardParams()
    p.rows, p.dim = x2.shape
    p.in_type = _lib.QA_IN_F16 if x.dtype == torch.float16 else _lib.QA_IN_F32
    p.scale = float(scale)
    p.x_row_stride, p.out_row_stride = x2.stride(0) if x2.shape[0] > 1 else dim, dim
    p.x, p.out = ptr(x2), ptr(out)
    with torch.cuda.device(x.device):
        st = _lib.lib().qa_hadamard_quant(ct.byref(p), _lib.current_stream(x.device))
    _lib.check(st, "hadamard_quant")
    return out.reshape(shape)


def qlayer_normgated_fwd(x, weight, bias, eps, q_z=None, z_scale=None, static_out_scale=None,
                         use_float16_output=False, group_size=None, norm_before_gate=True, is_rms_norm=True):
    """Gated RMS norm of fp16 rows (``_qlayer_normgated_fwd``, quamba/triton/quant_normgated.py:85-134).
    x fp16 (M, N); q_z int8 (M, N) or None.  Returns (out, per_token_scale): out fp16, or int8 with the
    static scale, or int8 with one dynamic scale per (row, group) in per_token_scale[(group, row)]."""
    _require(x.dtype == torch.float16 and x.dim() == 2, "x must be fp16 (M, N)")
    _require_gpu(x, "x")
    if bias is not None or not is_rms_norm:
        raise NotImplementedError("only the bias-free RMS norm is implemented")
    M, N = x.shape
    group_size = N if group_size is None else group_size
    _require(N % group_size == 0, "N must be divisible by group_size")
    _require(x.stride(-1) == 1, "x must be contiguous along the last dimension")
    _require(weight.dtype == torch.float16 and tuple(weight.shape) == (N,) and weight.stride(-1) == 1 and weight.is_cuda,
             "weight must be a contiguous fp16 GPU tensor of shape (N,)")
    if q_z is not None:
        _require(q_z.dtype == torch.int8 and tuple(q_z.shape) == (M, N) and q_z.stride(-1) == 1 and q_z.is_cuda,
                 "q_z must be an int8 GPU tensor of shape (M, N), contiguous along the last dimension")
    ngroups = N // group_size
    out = torch.empty((M, N), dtype=torch.float16 if use_float16_output else torch.int8, device=x.device)
    per_token_scale = torch.empty((ngroups * M,), dtype=torch.float32, device=x.device)
    p = _lib.QaNormGatedParams()
    p.rows, p.dim, p.group_size = M, N, group_size
    p.norm_before_gate = int(bool(norm_before_gate))
    p.out_mode = 0 if use_float16_output else (1 if static_out_scale is not None else 2)
    p.eps = float(eps)
    p.z_scale = float(z_scale) if z_scale is not None else 0.0
    p.out_scale = float(static_out_scale) if static_out_scale is not None else 0.0
    p.x_row_stride, p.out_row_stride = x.stride(0) if M > 1 else N, N
    p.z_row_stride = (q_z.stride(0) if M > 1 else N) if q_z is not None else 0
    p.x, p.weight, p.qz, p.out, p.dyn_scale = ptr(x), ptr(weight), ptr(q_z), ptr(out), ptr(per_token_scale)
    with torch.cuda.device(x.device):
        st = _lib.lib().qa_rmsnorm_gated(ct.byref(p), _lib.current_stream(x.device))
    _lib.check(st, "rmsnorm_gated")
    return out, per_token_scale


def normgated_hadamard_supported(dim, group_size):
    """Shapes for which the gated norm and the Hadamard transform run as one kernel."""
    return dim in (2048, 4096, 8192) and group_size in (512, 1024, 2048) and dim % group_size == 0


def qlayer_normgated_hadamard_quant(x, weight, eps, had_scale, q_z=None, z_scale=None, group_size=None,
                                    norm_before_gate=True):
    """hadamard_quant(qlayer_normgated_fwd(..., use_float16_output=True)[0], had_scale) in one kernel, bit for
    bit (QRMSNormGated.forward, quamba/qNorm.py:93-177, followed by the transform in front of out_proj,
    quamba/qHadamard.py).  x fp16 (M, N); q_z int8 (M, N) or None.  Returns int8 (M, N).  Only for shapes
    accepted by ``normgated_hadamard_supported``."""
    _require(x.dtype == torch.float16 and x.dim() == 2, "x must be fp16 (M, N)")
    _require_gpu(x, "x")
    M, N = x.shape
    group_size = N if group_size is None else group_size
    _require(normgated_hadamard_supported(N, group_size), "shape not covered by the fused kernel")
    _require(x.stride(-1) == 1, "x must be contiguous along the last dimension")
    _require(weight.dtype == torch.float16 and tuple(weight.shape) == (N,) and weight.stride(-1) == 1 and weight.is_cuda,
             "weight must be a contiguous fp16 GPU tensor of shape (N,)")
    if q_z is not None:
        _require(q_z.dtype == torch.int8 and tuple(q_z.shape) == (M, N) and q_z.stride(-1) == 1 and q_z.is_cuda,
                 "q_z must be an int8 GPU tensor of shape (M, N), contiguous along the last dimension")
    out = torch.empty((M, N), dtype=torch.int8, device=x.device)
    n = _lib.QaNormGatedParams()
    n.rows, n.dim, n.group_size = M, N, group_size
    n.norm_before_gate = int(bool(norm_before_gate))
    n.out_mode = 0
    n.eps = float(eps)
    n.z_scale = float(z_scale) if z_scale is not None else 0.0
    n.x_row_stride = x.stride(0) if M > 1 else N
    n.z_row_stride = (q_z.stride(0) if M > 1 else N) if q_z is not None else 0
    n.x, n.weight, n.qz = ptr(x), ptr(weight), ptr(q_z)
    h = _lib.QaHadamardParams()
    h.rows, h.dim = M, N
    h.scale = float(had_scale)
    h.out_row_stride = N
    h.out = ptr(out)
    with torch.cuda.device(x.device):
        st = _lib.lib().qa_rmsnorm_gated_hadamard_quant(ct.byref(n), ct.byref(h), _lib.current_stream(x.device))
    _lib.check(st, "rmsnorm_gated_hadamard_quant")
    return out


def sscan_fwd(u, scale_u, delta, scale_delta, A, scale_A, B, scale_B, C, scale_C, scale_ssm_state,
              D=None, scale_D=None, z=None, scale_z=None, delta_bias=None, scale_delta_bias=None,
              delta_softplus=False, state_dtype=torch.int8):
    """Selective scan over int8 inputs.

    u, delta, z: int8 (batch, dim, seqlen) with unit stride along seqlen; A: int8 (dim, dstate) holding
    A_log; B, C: int8 (batch, n_groups, dstate, seqlen).  Returns (out fp16 (batch, seqlen, dim),
    x) where x is the state after the last step: int8 (batch, dim, 1, dstate) by default (the
    reference's per-chunk state tensor, one chunk) or fp32 with ``state_dtype=torch.float32``.
    """
    _require(u.dtype == torch.int8 and A.dtype == torch.int8, "u and A must be int8")
    _require(delta.dtype == torch.int8 and B.dtype == torch.int8 and C.dtype == torch.int8,
             "delta, B and C must be int8")
    for t, n in ((u, "u"), (delta, "delta"), (A, "A"), (B, "B"), (C, "C")):
        _require_gpu(t, n)
    if B.dim() < 3 or C.dim() < 3:
        raise NotImplementedError("Must be input-dependent B and C")
    _require(u.dim() == 3, "u must have shape (batch, dim, seqlen)")
    batch, dim, seqlen = u.shape
    dstate = A.shape[1]
    _require(dstate <= 256, "quant_sscan only supports state dimension <= 256")
    _require(tuple(delta.shape) == (batch, dim, seqlen), "delta must have shape (batch, dim, seqlen)")
    _require(tuple(A.shape) == (dim, dstate), "A must have shape (dim, dstate)")
    n_groups = B.shape[1]
    _require(tuple(B.shape) == (batch, n_groups, dstate, seqlen) and tuple(C.shape) == tuple(B.shape),
             "B and C must have shape (batch, n_groups, dstate, seqlen)")
    for t, n in ((u, "u"), (delta, "delta"), (B, "B"), (C, "C")):
        _require(t.stride(-1) == 1 or t.size(-1) == 1, f"{n} must have unit stride along seqlen")
    for s, n in ((scale_u, "scale_u"), (scale_delta, "scale_delta"), (scale_A, "scale_A"), (scale_B, "scale_B"),
                 (scale_C, "scale_C")):
        _scale1(s, n)
    p = _lib.QaSScanParams()
    if D is not None:
        _require(D.dtype == torch.int8 and D.is_cuda and tuple(D.shape) == (dim,) and D.stride(-1) == 1,
                 "D must be a contiguous int8 GPU tensor of shape (dim,)")
        _scale1(scale_D, "scale_D")
        p.D, p.scale_D = ptr(D), ptr(scale_D)
    if delta_bias is not None:
        _require(delta_bias.dtype == torch.int8 and delta_bias.is_cuda and tuple(delta_bias.shape) == (dim,)
                 and delta_bias.stride(-1) == 1, "delta_bias must be a contiguous int8 GPU tensor of shape (dim,)")
        _scale1(scale_delta_bias, "scale_delta_bias")
        p.delta_bias, p.scale_delta_bias = ptr(delta_bias), ptr(scale_delta_bias)
    if z is not None:
        _require(z.dtype == torch.int8 and z.is_cuda and tuple(z.shape) == (batch, dim, seqlen),
                 "z must be an int8 GPU tensor of shape (batch, dim, seqlen)")
        _require(z.stride(-1) == 1 or z.size(-1) == 1, "z must have unit stride along seqlen")
        _scale1(scale_z, "scale_z")
        p.z, p.scale_z = ptr(z), ptr(scale_z)
        p.z_batch_stride, p.z_d_stride = z.stride(0), z.stride(1)
    out = torch.empty((batch, seqlen, dim), dtype=torch.float16, device=u.device)
    x = torch.empty((batch, dim, 1, dstate), dtype=state_dtype, device=u.device)
    if state_dtype == torch.int8:
        _scale1(scale_ssm_state, "scale_ssm_state")
        p.last_state_i8, p.scale_ssm_state = ptr(x), ptr(scale_ssm_state)
    else:
        _require(state_dtype == torch.float32, "state_dtype must be torch.int8 or torch.float32")
        p.last_state_f32 = ptr(x)
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups = batch, dim, seqlen, dstate, n_groups
    p.delta_softplus = int(bool(delta_softplus))
    p.u_batch_stride, p.u_d_stride = u.stride(0), u.stride(1)
    p.delta_batch_stride, p.delta_d_stride = delta.stride(0), delta.stride(1)
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = B.stride(0), B.stride(1), B.stride(2)
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = C.stride(0), C.stride(1), C.stride(2)
    p.A_d_stride, p.A_dstate_stride = A.stride(0), A.stride(1)
    p.out_batch_stride, p.out_l_stride, p.out_d_stride = out.stride()
    p.u, p.delta, p.A_log, p.B, p.C, p.out = ptr(u), ptr(delta), ptr(A), ptr(B), ptr(C), ptr(out)
    p.scale_u, p.scale_delta, p.scale_A = ptr(scale_u), ptr(scale_delta), ptr(scale_A)
    p.scale_B, p.scale_C = ptr(scale_B), ptr(scale_C)
    p.mapping = SSCAN_MAPPING
    segments = _sscan_segments(batch, dim, seqlen)
    with torch.cuda.device(u.device):
        stream = _lib.current_stream(u.device)
        if segments <= 1:
            st = _lib.lib().qa_sscan_fwd(ct.byref(p), stream)
        else:
            # One sequence alone leaves most of the chip idle (a wave walks all of its steps), so it is scanned as
            # `segments` pieces side by side: every piece from a zero state, which also yields each piece's end
            # state and the sum of its step sizes; then the pieces after the first once more, each from the state
            # its predecessors chain up to.  Twice the arithmetic on `segments` times the waves.
            seg = seqlen // segments
            local = torch.empty((segments, dim, dstate), dtype=torch.float32, device=u.device)
            dt_sum = torch.empty((segments, dim), dtype=torch.float32, device=u.device)
            p1 = _lib.QaSScanParams.from_buffer_copy(p)
            p1.batch, p1.seqlen = segments, seg
            p1.u_batch_stride = p1.delta_batch_stride = p1.z_batch_stride = seg
            p1.B_batch_stride = p1.C_batch_stride = seg
            p1.out_batch_stride = seg * out.stride(1)
            p1.last_state_i8, p1.last_state_f32, p1.dt_sum_out = None, ptr(local), ptr(dt_sum)
            st = _lib.lib().qa_sscan_fwd(ct.byref(p1), stream)
            if st == 0:
                tail = torch.empty((segments - 1, dim, dstate), dtype=state_dtype, device=u.device)
                p2 = _lib.QaSScanParams.from_buffer_copy(p1)
                p2.batch = segments - 1
                p2.u, p2.delta = u.data_ptr() + seg, delta.data_ptr() + seg
                p2.B, p2.C = B.data_ptr() + seg, C.data_ptr() + seg
                if z is not None:
                    p2.z = z.data_ptr() + seg
                p2.out = out.data_ptr() + seg * out.stride(1) * 2
                p2.dt_sum_out, p2.carry_dt_sum, p2.carry_state, p2.carry_first = None, ptr(dt_sum), ptr(local), 1
                if state_dtype == torch.int8:
                    p2.last_state_i8, p2.last_state_f32 = ptr(tail), None
                else:
                    p2.last_state_i8, p2.last_state_f32 = None, ptr(tail)
                st = _lib.lib().qa_sscan_fwd(ct.byref(p2), stream)
                x = tail[-1].reshape(1, dim, 1, dstate)
    _lib.check(st, "sscan_fwd")
    return out, x


# A single sequence of at least this many steps is scanned in segments (see sscan_fwd); 0 disables it.
SSCAN_SEGMENT_MIN_STEPS = 1024
# QaSScanParams.mapping of every call: 0 lets the library choose; tests set sscan_mapping(lanes, arg) to reach each
# kernel variant on one shape.
SSCAN_MAPPING = 0


def sscan_mapping(lanes, arg):
    """QA_SSCAN_MAPPING(lanes per channel, waves per workgroup); lanes == 0: the launch with two kinds of
    workgroup, ``arg`` 64-channel workgroups per batch entry taking four lanes per channel."""
    return 0x40000000 | (int(lanes) << 20) | int(arg)


def sscan_chosen_mapping(batch, dim, dstate, n_groups=1):
    """(lanes per channel, argument) of the mapping qa_sscan_fwd takes for these sizes on the current device
    (qa_sscan_chosen_mapping); lanes == 0 is the launch with two kinds of workgroup, the argument then being the
    number of 64-channel workgroups per batch entry with four lanes per channel.  None for d_state above 16."""
    p = _lib.QaSScanParams()
    p.batch, p.dim, p.dstate, p.n_groups = batch, dim, dstate, n_groups
    code = _lib.lib().qa_sscan_chosen_mapping(ct.byref(p))
    if code < 0:
        _lib.check(code, "sscan_chosen_mapping")
    return None if code == 0 else ((code >> 20) & 0xff, code & 0xfffff)


def _sscan_segments(batch, dim, seqlen):
    if batch != 1 or not SSCAN_SEGMENT_MIN_STEPS or seqlen < SSCAN_SEGMENT_MIN_STEPS:
        return 1
    for segments in (8, 4, 2):
        # equal pieces whose rows keep the 16-byte alignment of the whole, at least 128 steps each
        if seqlen % (segments * 16) == 0 and seqlen // segments >= 128:
            return segments
    return 1



def sscan_update(state, q_x, x_scale, q_dt, dt_scale, q_A_log, A_log_scale, ssm_state_scale, q_B, B_scale,
                 q_C, C_scale, q_D=None, D_scale=None, q_z=None, z_scale=None, dt_bias=None, dt_bias_scale=None,
                 dt_softplus=False, x_head_group_range=None, x_dim_group_range=None, _conv_step=None):
    """One recurrence step; ``state`` (int8 with ssm_state_scale, or fp32) is updated in place.

    Shapes as quamba/triton/selective_state_update.py:129-160: state (batch, dim, dstate) or
    (batch, nheads, dim, dstate); q_x, q_dt, q_z (batch, dim) or (batch, nheads, dim); q_A_log
    (dim, dstate) or (nheads, dim, dstate); q_B, q_C (batch, dstate) or (batch, ngroups, dstate);
    q_D, dt_bias (dim) or (nheads, dim).  dt_bias is int8 with dt_bias_scale, or fp16/fp32 without.
    With x_head_group_range / x_dim_group_range the scales are the grouped ones of
    quamba2_sscan_update_triton (:365-478).  Returns out fp16 shaped like q_x.
    """
    has_heads = state.dim() > 3
    if state.dim() == 3:
        state = state.unsqueeze(1)
    q_x = q_x.unsqueeze(1) if q_x.dim() == 2 else q_x
    q_dt = q_dt.unsqueeze(1) if q_dt.dim() == 2 else q_dt
    q_A_log = q_A_log.unsqueeze(0) if q_A_log.dim() == 2 else q_A_log
    q_B = q_B.unsqueeze(1) if q_B.dim() == 2 else q_B
    q_C = q_C.unsqueeze(1) if q_C.dim() == 2 else q_C
    if q_D is not None and q_D.dim() == 1:
        q_D = q_D.unsqueeze(0)
    if q_z is not None and q_z.dim() == 2:
        q_z = q_z.unsqueeze(1)
    if dt_bias is not None and dt_bias.dim() == 1:
        dt_bias = dt_bias.unsqueeze(0)
    batch, nheads, dim, dstate = state.shape
    ngroups = q_B.shape[1]
    _require(state.dtype in (torch.int8, torch.float32), "state must be int8 or fp32")
    _require_gpu(state, "state")
    _require(tuple(q_x.shape) == (batch, nheads, dim), "x must have shape (batch, [nheads,] dim)")
    _require(tuple(q_dt.shape) == tuple(q_x.shape), "dt must have the shape of x")
    _require(tuple(q_A_log.shape) == (nheads, dim, dstate), "A_log must have shape ([nheads,] dim, dstate)")
    _require(nheads % ngroups == 0, "nheads must be divisible by ngroups")
    _require(tuple(q_B.shape) == (batch, ngroups, dstate) and tuple(q_C.shape) == tuple(q_B.shape),
             "B and C must have shape (batch, [ngroups,] dstate)")
    for t in (q_x, q_dt, q_A_log, q_B, q_C):
        _require(t.dtype == torch.int8 and t.is_cuda, "x, dt, A_log, B and C must be int8 GPU tensors")
    _require(dstate <= 256, "state dimension must be <= 256")
    out = torch.empty(q_x.shape, dtype=torch.float16, device=q_x.device)
    p = _lib.QaSsmUpdateParams()
    p.batch, p.nheads, p.dim, p.dstate, p.ngroups = batch, nheads, dim, dstate, ngroups
    p.dt_softplus = int(bool(dt_softplus))
    p.state_is_fp32 = int(state.dtype == torch.float32)
    (p.state_batch_stride, p.state_head_stride, p.state_dim_stride, p.state_dstate_stride) = state.stride()
    p.x_batch_stride, p.x_head_stride, p.x_dim_stride = q_x.stride()
    p.dt_batch_stride, p.dt_head_stride, p.dt_dim_stride = q_dt.stride()
    p.A_head_stride, p.A_dim_stride, p.A_dstate_stride = q_A_log.stride()
    p.B_batch_stride, p.B_group_stride, p.B_dstate_stride = q_B.stride()
    p.C_batch_stride, p.C_group_stride, p.C_dstate_stride = q_C.stride()
    p.out_batch_stride, p.out_head_stride, p.out_dim_stride = out.stride()
    p.state, p.x, p.dt, p.A_log, p.B, p.C, p.out = (ptr(state), ptr(q_x), ptr(q_dt), ptr(q_A_log), ptr(q_B),
                                                   ptr(q_C), ptr(out))
    keep = []

    def f32(t):
        if not (t.dtype == torch.float32 and t.device == q_x.device and t.is_contiguous()):
            t = t.to(device=q_x.device, dtype=torch.float32).contiguous()
            keep.append(t)
        return t.data_ptr()

    p.x_scale, p.dt_scale, p.A_log_scale = f32(x_scale), f32(dt_scale), f32(A_log_scale)
    p.B_scale, p.C_scale = f32(B_scale), f32(C_scale)
    if not p.state_is_fp32:
        p.state_scale = f32(ssm_state_scale)
    if x_head_group_range is not None:
        _require(x_head_group_range.dtype == torch.int32 and x_dim_group_range.dtype == torch.int32,
                 "group ranges must be int32")
        _require(x_head_group_range.dim() == 2 and x_dim_group_range.dim() == 3,
                 "x_head_group_range must be [ngroups, nhead_groups], x_dim_group_range [ngroups, nhead_groups, ndim_groups]")
        p.nhead_groups, p.ndim_groups = x_head_group_range.shape[1], x_dim_group_range.shape[2]
        _require(x_scale.numel() == ngroups * p.nhead_groups * p.ndim_groups, "x_scale has the wrong number of groups")
        if not p.state_is_fp32:
            _require(tuple(ssm_state_scale.shape) == (ngroups, p.nhead_groups, p.ndim_groups, dstate),
                     "ssm_state_scale must be [ngroups, nhead_groups, ndim_groups, dstate]")
        hr, dr = x_head_group_range.contiguous(), x_dim_group_range.contiguous()
        keep += [hr, dr]
        p.x_head_group_range, p.x_dim_group_range = ptr(hr), ptr(dr)
    if q_D is not None:
        _require(tuple(q_D.shape) == (nheads, dim) and q_D.dtype == torch.int8, "D must be int8 ([nheads,] dim)")
        p.D, p.D_scale = ptr(q_D), f32(D_scale)
        p.D_head_stride, p.D_dim_stride = q_D.stride()
    if q_z is not None:
        _require(tuple(q_z.shape) == tuple(q_x.shape) and q_z.dtype == torch.int8, "z must be int8 shaped like x")
        p.z, p.z_scale = ptr(q_z), f32(z_scale)
        p.z_batch_stride, p.z_head_stride, p.z_dim_stride = q_z.stride()
    if dt_bias is not None:
        _require(tuple(dt_bias.shape) == (nheads, dim), "dt_bias must have shape ([nheads,] dim)")
        if dt_bias.dtype == torch.int8:
            p.dt_bias_scale = f32(dt_bias_scale)
        else:
            if dt_bias.dtype != torch.float16:
                dt_bias = dt_bias.to(torch.float16)
                keep.append(dt_bias)
            p.dt_bias_is_fp16 = 1
        p.dt_bias = ptr(dt_bias)
        p.dt_bias_head_stride, p.dt_bias_dim_stride = dt_bias.stride()
    with torch.cuda.device(q_x.device):
        if _conv_step is not None:
            # q_x is the buffer the conv step of the same launch writes (see mamba1_decode_step)
            st = _lib.lib().qa_mamba1_decode_step(ct.byref(_conv_step), ct.byref(p), _lib.current_stream(q_x.device))
        else:
            st = _lib.lib().qa_ssm_state_update(ct.byref(p), _lib.current_stream(q_x.device))
    _lib.check(st, "mamba1_decode_step" if _conv_step is not None else "ssm_state_update")
    return out if has_heads else out.squeeze(1)


# ----------------------------------------------------------------------------------------------
# W8A8 linear
# ----------------------------------------------------------------------------------------------
def _gemm_w8a8(c, a, w_nk, a_scales, b_scales, alpha=None, round_half_away=False):
    """c (M,N) row-major <- a (M,K) x w_nk (N,K)^T, both K-contiguous."""
    _require(a.dtype == torch.int8 and w_nk.dtype == torch.int8, "a and b must be int8")
    for t, n in ((a, "a"), (w_nk, "b"), (c, "c")):
        _require_gpu(t, n)
    _require(c.dtype in (torch.int8, torch.float16, torch.bfloat16), "c must be int8, fp16 or bf16")
    M, K = a.shape
    N = w_nk.shape[0]
    _require(w_nk.shape[1] == K and tuple(c.shape) == (M, N), "shape mismatch: c (M,N) = a (M,K) x b (K,N)")
    _require(a.stride(1) == 1 and c.stride(1) == 1, "a and c must be row-major")
    _require(w_nk.stride(1) == 1, "b must be column-major (K contiguous)")
    _require(a.stride(0) % 16 == 0 and w_nk.stride(0) % 16 == 0 and K % 16 == 0,
             "row strides of a and b and K must be multiples of 16")
    p = _lib.QaGemmW8A8Params()
    p.m, p.n, p.k = M, N, K
    p.out_type = {torch.int8: _lib.QA_OUT_I8, torch.float16: _lib.QA_OUT_F16, torch.bfloat16: _lib.QA_OUT_BF16}[c.dtype]
    p.round_mode = _lib.QA_ROUND_HALF_AWAY if round_half_away else _lib.QA_ROUND_RNE
    p.lda, p.ldw, p.ldd = a.stride(0), w_nk.stride(0), c.stride(0)
    p.a, p.w, p.d = ptr(a), ptr(w_nk), ptr(c)
    if alpha is not None:
        p.use_alpha, p.alpha = 1, float(alpha)
    else:
        for s, n, full in ((a_scales, "a_scales", M), (b_scales, "b_scales", N)):
            _require(s.dtype == torch.float32 and s.is_cuda and s.is_contiguous(), f"{n} must be contiguous fp32 on the GPU")
            _require(s.numel() in (1, full), f"{n} must have 1 or {full} elements")
        p.a_scale, p.w_scale = ptr(a_scales), ptr(b_scales)
        p.a_scale_numel, p.w_scale_numel = a_scales.numel(), b_scales.numel()
    with torch.cuda.device(a.device):
        st = _lib.lib().qa_gemm_w8a8(ct.byref(p), _lib.current_stream(a.device))
    _lib.check(st, "gemm_w8a8")
    return c


def scaled_mm_dq(c, a, b, a_scales, b_scales):
    """c = cast(a_scales * (b_scales * (a @ b))) with a int8 (M,K) row-major, b int8 (K,N) column-major
    (b.stride(0) == 1), scales fp32 with 1 or M / 1 or N elements; c int8 (round-half-even,
    saturating), fp16 or bf16, written in place.  Interface of cutlass_scaled_mm_dq."""
    _require(b.dim() == 2 and b.stride(0) == 1, "b must be column-major")
    return _gemm_w8a8(c, a, b.t(), a_scales, b_scales)


def scaled_mv_dq(y, w, x, alpha, beta=0.0):
    """y (1,N) = cast(alpha * (x (1,K) @ w (N,K)^T)); interface of cutlass_scaled_mv_dq (beta must be 0)."""
    _require(float(beta) == 0.0, "beta != 0 is not supported")
    return _gemm_w8a8(y, x, w, None, None, alpha=alpha)


def w8a8o8_gemv(y, w, x, b_scales, a_scale):
    """y (1,N) int8 = sat8(roundf(b_scales[n] * a_scale * (x @ w^T))); interface of w8a8o8_gemv.
    The reference multiplies b_scales[n] * a_scale first (quant_linear_fwd_gemv_kernel.cuh:56-60); the two scale
    operands are therefore passed swapped so that the same product is formed."""
    return _gemm_w8a8(y, x, w, a_scale, b_scales, round_half_away=True)


# ----------------------------------------------------------------------------------------------
# W4A8 linear
# ----------------------------------------------------------------------------------------------
# from this many activation rows on the 4-bit weights are expanded once per call into a scratch buffer: the fused
# kernel expands them again in every band of 256 rows (measured: 512 rows 81 vs 97 us, 1024 rows 137 vs 105 us at
# 4096 -> 18560)
W4A8_EXPAND_ONCE_ROWS = 1024


def _w4a8_gemm(a, b_q_weight, s_tok, s_ch, s_group, m, n, k, output_transpose, out_dtype):
    _require(a.dtype == torch.int8 and a.is_cuda and a.dim() == 2 and a.is_contiguous(), "a must be a contiguous int8 GPU matrix")
    _require(tuple(a.shape) == (m, k), "a must have shape (m, k)")
    _require(b_q_weight.dtype == torch.uint8 and b_q_weight.is_cuda and tuple(b_q_weight.shape) == (n, k // 2)
             and b_q_weight.is_contiguous(), "b_q_weight must be uint8 (n, k/2) in this library's packing")
    _require(k % 128 == 0, "k must be a multiple of 128")
    _require(s_ch.dtype == torch.float32 and s_ch.is_cuda and s_ch.numel() == n, "s_ch must be fp32 with n elements")
    _require(s_tok.dtype == torch.float32 and s_tok.is_cuda and s_tok.numel() in (1, m),
             "s_tok must be fp32 with 1 or m elements")
    grouped = s_group is not None and s_group.numel() > 0
    if grouped:
        _require(s_group.dtype == torch.float16 and s_group.is_cuda and tuple(s_group.shape) == (k // 128, n)
                 and s_group.is_contiguous(), "s_group must be contiguous fp16 (k/128, n)")
    d = torch.empty((n, m) if output_transpose else (m, n), dtype=out_dtype, device=a.device)
    p = _lib.QaGemmW4A8Params()
    p.m, p.n, p.k = m, n, k
    p.group_size = 128 if grouped else -1
    p.out_type = _lib.QA_OUT_I8 if out_dtype == torch.int8 else _lib.QA_OUT_F16
    p.tok_scale_numel = s_tok.numel()
    p.output_transpose = int(bool(output_transpose))
    p.lda, p.ldd = a.stride(0), d.stride(0)
    s_ch_c, s_tok_c = s_ch.contiguous(), s_tok.contiguous()
    p.a, p.w_packed, p.s_group = ptr(a), ptr(b_q_weight), ptr(s_group) if grouped else None
    p.s_channel, p.s_token, p.d = ptr(s_ch_c), ptr(s_tok_c), ptr(d)
    w8 = None
    if m >= W4A8_EXPAND_ONCE_ROWS:
        # many rows: scratch for the weights expanded to int8 once (see QaGemmW4A8Params.w8_workspace)
        w8 = torch.empty(n * k, dtype=torch.int8, device=a.device)
        p.w8_workspace, p.w8_workspace_bytes = ptr(w8), w8.numel()
    with torch.cuda.device(a.device):
        st = _lib.lib().qa_gemm_w4a8(ct.byref(p), _lib.current_stream(a.device))
    _lib.check(st, "gemm_w4a8")
    return d


def w4a8o16_gemm(a, b_q_weight, s_tok, s_ch, s_group, workspace, m, n, k, output_transpose=False):
    """fp16 (m, n) [or (n, m)] = ((a @ dequant(b)^T) * s_ch[n]) * s_tok[m|0].  ``workspace`` is accepted for
    interface compatibility and unused (no cross-workgroup reduction is needed)."""
    return _w4a8_gemm(a, b_q_weight, s_tok, s_ch, s_group, m, n, k, output_transpose, torch.float16)


def w4a8o8_gemm(a, b_q_weight, s_tok, s_ch, s_group, workspace, m, n, k, output_transpose=False):
    """int8 variant: round-half-even, saturating."""
    return _w4a8_gemm(a, b_q_weight, s_tok, s_ch, s_group, m, n, k, output_transpose, torch.int8)


# ----------------------------------------------------------------------------------------------
# Mamba2 SSD chunk scan
# ----------------------------------------------------------------------------------------------
def ssd_chunk_scan_combined_fwd(q_x, x_scale, q_dt, dt_scale, q_A_log, A_log_scale, q_B, B_scale, q_C, C_scale,
                                ssm_state_scale, chunk_size, q_D=None, D_scale=None, q_z=None, z_scale=None,
                                dt_bias=None, initial_states=None, seq_idx=None, cu_seqlens=None, dt_softplus=False,
                                dt_limit=(0.0, float("inf")), x_head_group_range=None, x_dim_group_range=None,
                                final_state_dtype=torch.int8, return_workspace=False, static_scratch=False):
    """Quantized SSD forward; interface of _quant_mamba_chunk_scan_combined_fwd and, with the group
    ranges, of _quamba2_mamba_chunk_scan_combined_fwd (quamba/triton/quant_ssd_combined.py:11-166).

    q_x int8 (batch, seqlen, nheads, headdim); q_dt int8 (batch, seqlen, nheads), or fp32 holding the
    already processed step sizes; q_A_log int8 (nheads); q_B, q_C int8 (batch, seqlen, ngroups,
    dstate); q_D int8 (nheads) or (nheads, headdim); dt_bias fp16 (nheads).
    Returns (out fp16 like q_x, final_states (batch, nheads, headdim, dstate) int8 or fp32).
    With ``static_scratch`` the intermediates live in the library's fixed device buffer instead of a workspace
    allocated here (qa_ssd_chunk_scan_fwd_noalloc: for callers that must not allocate; calls on one GPU must
    not overlap); problems that need more than the buffer holds raise RuntimeError.
    """
    if initial_states is not None:
        raise NotImplementedError("initial_states is not supported")
    if seq_idx is not None:
        raise NotImplementedError("seq_idx is not supported")
    if cu_seqlens is not None:
        raise NotImplementedError("Only supports `cu_seqlens=None`")
    _require(q_x.dtype == torch.int8 and q_x.is_cuda and q_x.dim() == 4, "q_x must be int8 (batch, seqlen, nheads, headdim) on the GPU")
    batch, seqlen, nheads, headdim = q_x.shape
    _require(q_B.dtype == torch.int8 and q_B.dim() == 4 and q_B.shape[:2] == (batch, seqlen), "q_B must be int8 (batch, seqlen, ngroups, dstate)")
    ngroups, dstate = q_B.shape[2], q_B.shape[3]
    _require(tuple(q_C.shape) == tuple(q_B.shape) and q_C.dtype == torch.int8, "q_C must match q_B")
    _require(nheads % ngroups == 0, "nheads must be divisible by ngroups")
    _require(tuple(q_dt.shape) == (batch, seqlen, nheads) and q_dt.dtype in (torch.int8, torch.float32),
             "q_dt must be int8 or fp32 (batch, seqlen, nheads)")
    _require(tuple(q_A_log.shape) == (nheads,) and q_A_log.dtype == torch.int8, "q_A_log must be int8 (nheads,)")
    dev = q_x.device
    keep = []

    def f32(t):
        t = torch.as_tensor(t, device=dev).to(torch.float32).contiguous()
        keep.append(t)
        return ptr(t)

    # The matrix-core kernels are built for head dimensions that are multiples of 64, 64 or 128 states and chunks of
    # 64, 128 or 256 steps; the library runs every other shape on general kernels.  Fewer than 128 states (the
    # reference's tests use 16) with an otherwise fast shape run as 64 or 128 with zero codes in the added B and C
    # columns: those states stay zero and add exactly nothing.
    dstate_given = dstate
    if headdim % 64 == 0 and chunk_size in (64, 128, 256) and dstate not in (64, 128) and dstate < 128:
        dstate = 64 if dstate < 64 else 128
        q_B = torch.nn.functional.pad(q_B, (0, dstate - dstate_given))
        q_C = torch.nn.functional.pad(q_C, (0, dstate - dstate_given))
    q_x, q_B, q_C, q_dt = q_x.contiguous(), q_B.contiguous(), q_C.contiguous(), q_dt.contiguous()
    p = _lib.QaSsdParams()
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups = batch, seqlen, nheads, headdim, dstate, ngroups
    p.chunk_size = chunk_size
    p.dt_softplus = int(bool(dt_softplus))
    p.dt_is_fp32 = int(q_dt.dtype == torch.float32)
    p.dt_min, p.dt_max = float(dt_limit[0]), float(min(dt_limit[1], 3.0e38))
    p.x, p.dt, p.A_log, p.B, p.C = ptr(q_x), ptr(q_dt), ptr(q_A_log.contiguous()), ptr(q_B), ptr(q_C)
    p.x_scale, p.A_log_scale, p.B_scale, p.C_scale = f32(x_scale), f32(A_log_scale), f32(B_scale), f32(C_scale)
    if not p.dt_is_fp32:
        p.dt_scale = f32(dt_scale)
        if dt_bias is not None:
            b16 = dt_bias.to(device=dev, dtype=torch.float16).contiguous()
            keep.append(b16)
            p.dt_bias = ptr(b16)
    if x_head_group_range is not None:
        _require(x_head_group_range.dtype == torch.int32 and x_dim_group_range.dtype == torch.int32, "group ranges must be int32")
        hr, dr = x_head_group_range.contiguous(), x_dim_group_range.contiguous()
        keep += [hr, dr]
        p.nhead_groups, p.ndim_groups = hr.shape[1], dr.shape[2]
        p.x_head_group_range, p.x_dim_group_range = ptr(hr), ptr(dr)
        _require(keep[0].numel() == ngroups * p.nhead_groups * p.ndim_groups, "x_scale has the wrong number of groups")
    if q_D is not None:
        _require(tuple(q_D.shape) in ((nheads,), (nheads, headdim)) and q_D.dtype == torch.int8, "q_D must be int8 (nheads[, headdim])")
        qd = q_D.contiguous()
        keep.append(qd)
        p.D, p.D_scale, p.D_has_hdim = ptr(qd), f32(D_scale), int(q_D.dim() == 2)
    if q_z is not None:
        _require(tuple(q_z.shape) == tuple(q_x.shape) and q_z.dtype == torch.int8, "q_z must be int8 shaped like q_x")
        qz = q_z.contiguous()
        keep.append(qz)
        p.z, p.z_scale = ptr(qz), f32(z_scale)
    out = torch.empty(q_x.shape, dtype=torch.float16, device=dev)
    final = torch.empty((batch, nheads, headdim, dstate), dtype=final_state_dtype, device=dev)
    p.out, p.final_states = ptr(out), ptr(final)
    p.final_state_is_fp32 = int(final_state_dtype == torch.float32)
    if not p.final_state_is_fp32:
        _require(final_state_dtype == torch.int8, "final_state_dtype must be torch.int8 or torch.float32")
        ssm_state_scale = torch.as_tensor(ssm_state_scale, device=dev).to(torch.float32)
        if p.nhead_groups:
            _require(tuple(ssm_state_scale.shape) == (ngroups, p.nhead_groups, p.ndim_groups, dstate_given),
                     "ssm_state_scale must be [ngroups, nhead_groups, ndim_groups, dstate]")
            if dstate != dstate_given:
                # the kernel walks the scale rows with the padded state count; the added states are zero, so
                # any finite scale serves for them
                ssm_state_scale = torch.nn.functional.pad(ssm_state_scale, (0, dstate - dstate_given), value=1.0)
        else:
            _require(ssm_state_scale.numel() == 1, "ssm_state_scale must have one element without group ranges")
        p.state_scale = f32(ssm_state_scale)
    lib = _lib.lib()
    nbytes = lib.qa_ssd_workspace_bytes(ct.byref(p))
    if nbytes <= 0:
        # an invalid request (the call reports which way), or an empty one (nothing to do)
        with torch.cuda.device(dev):
            _lib.check(lib.qa_ssd_chunk_scan_fwd(ct.byref(p), _lib.current_stream(dev)), "ssd_chunk_scan_fwd")
        if dstate != dstate_given:
            final = final[..., :dstate_given].contiguous()
        return (out, final, None) if return_workspace else (out, final)
    if static_scratch:
        _require(not return_workspace, "the library's own scratch buffer cannot be returned")
        with torch.cuda.device(dev):
            st = lib.qa_ssd_chunk_scan_fwd_noalloc(ct.byref(p), _lib.current_stream(dev))
        _lib.check(st, "ssd_chunk_scan_fwd_noalloc")
        ws = None
    else:
        ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
        p.workspace, p.workspace_bytes = ptr(ws), nbytes
        with torch.cuda.device(dev):
            st = lib.qa_ssd_chunk_scan_fwd(ct.byref(p), _lib.current_stream(dev))
        _lib.check(st, "ssd_chunk_scan_fwd")
    if dstate != dstate_given:
        final = final[..., :dstate_given].contiguous()
    if return_workspace:
        return out, final, ws
    return out, final

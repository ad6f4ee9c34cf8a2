"""ctypes binding of libquamba_amd.so (the C ABI declared in include/quamba_amd.h).

There is no fallback: if the shared library is missing or fails to load, importing an operator
raises.  Build it with ``python -m quamba_amd.build``.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libquamba_amd.so")

QA_OK = 0
ABI_VERSION = 2          # what qa_abi_version() of a matching library returns
QA_OUT_I8, QA_OUT_F16, QA_OUT_BF16 = 0, 1, 2
QA_ROUND_RNE, QA_ROUND_HALF_AWAY = 0, 1
QA_IN_F16, QA_IN_F32 = 0, 1

i32, i64, f32, vp = C.c_int32, C.c_int64, C.c_float, C.c_void_p


class QaConvParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("width", i32),
        ("silu_activation", i32), ("reserved0", i32),
        ("x_batch_stride", i64), ("x_c_stride", i64), ("x_l_stride", i64),
        ("out_batch_stride", i64), ("out_c_stride", i64), ("out_l_stride", i64),
        ("weight_c_stride", i64), ("weight_width_stride", i64),
        ("conv_state_batch_stride", i64), ("conv_state_c_stride", i64), ("conv_state_l_stride", i64),
        ("conv_state_len", i32), ("reserved1", i32),
        ("x", vp), ("weight", vp), ("bias", vp), ("out", vp), ("conv_state", vp),
        ("scale_x", f32), ("scale_w", f32), ("scale_b", f32), ("scale_out", f32),
        ("out_t", vp), ("out_t_batch_stride", i64), ("out_t_l_stride", i64),
    ]


class QaConv2Params(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("width", i32),
        ("silu_activation", i32),
        ("x_dim", i32), ("x_headdim", i32), ("d_state", i32), ("n_groups", i32),
        ("nhead_groups", i32), ("ndim_groups", i32), ("conv_state_len", i32),
        ("xBC_batch_stride", i64), ("xBC_l_stride", i64), ("xBC_c_stride", i64),
        ("x_batch_stride", i64), ("x_l_stride", i64), ("x_c_stride", i64),
        ("B_batch_stride", i64), ("B_l_stride", i64), ("B_c_stride", i64),
        ("C_batch_stride", i64), ("C_l_stride", i64), ("C_c_stride", i64),
        ("weight_c_stride", i64), ("weight_width_stride", i64),
        ("conv_state_batch_stride", i64), ("conv_state_c_stride", i64), ("conv_state_l_stride", i64),
        ("xBC", vp), ("weight", vp), ("bias", vp), ("x", vp), ("B", vp), ("C", vp), ("conv_state", vp),
        ("x_out_scales", vp), ("B_out_scales", vp), ("C_out_scales", vp),
        ("x_head_group_range", vp), ("x_dim_group_range", vp),
        ("scale_x", f32), ("scale_B", f32), ("scale_C", f32),
        ("scale_wx", f32), ("scale_wB", f32), ("scale_wC", f32),
        ("scale_bx", f32), ("scale_bB", f32), ("scale_bC", f32),
        ("reserved0", f32),
    ]


class QaHadamardParams(C.Structure):
    _fields_ = [
        ("rows", i32), ("dim", i32), ("in_type", i32), ("scale", f32),
        ("x_row_stride", i64), ("out_row_stride", i64),
        ("x", vp), ("out", vp),
    ]


class QaNormGatedParams(C.Structure):
    _fields_ = [
        ("rows", i32), ("dim", i32), ("group_size", i32), ("norm_before_gate", i32), ("out_mode", i32),
        ("eps", f32), ("z_scale", f32), ("out_scale", f32),
        ("x_row_stride", i64), ("z_row_stride", i64), ("out_row_stride", i64),
        ("x", vp), ("weight", vp), ("qz", vp), ("out", vp), ("dyn_scale", vp),
    ]


class QaSScanParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("dim", i32), ("seqlen", i32), ("dstate", i32),
        ("n_groups", i32), ("delta_softplus", i32),
        ("u_batch_stride", i64), ("u_d_stride", i64),
        ("delta_batch_stride", i64), ("delta_d_stride", i64),
        ("z_batch_stride", i64), ("z_d_stride", i64),
        ("B_batch_stride", i64), ("B_group_stride", i64), ("B_dstate_stride", i64),
        ("C_batch_stride", i64), ("C_group_stride", i64), ("C_dstate_stride", i64),
        ("A_d_stride", i64), ("A_dstate_stride", i64),
        ("out_batch_stride", i64), ("out_l_stride", i64), ("out_d_stride", i64),
        ("u", vp), ("delta", vp), ("A_log", vp), ("B", vp), ("C", vp), ("D", vp),
        ("delta_bias", vp), ("z", vp),
        ("scale_u", vp), ("scale_delta", vp), ("scale_A", vp), ("scale_B", vp), ("scale_C", vp),
        ("scale_D", vp), ("scale_delta_bias", vp), ("scale_z", vp), ("scale_ssm_state", vp),
        ("out", vp), ("last_state_i8", vp), ("last_state_f32", vp),
        ("dt_sum_out", vp), ("carry_dt_sum", vp), ("carry_state", vp), ("carry_first", i32), ("mapping", i32),
    ]


class QaSsmUpdateParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("nheads", i32), ("dim", i32), ("dstate", i32),
        ("ngroups", i32), ("dt_softplus", i32), ("state_is_fp32", i32), ("dt_bias_is_fp16", i32),
        ("nhead_groups", i32), ("ndim_groups", i32),
        ("state_batch_stride", i64), ("state_head_stride", i64), ("state_dim_stride", i64),
        ("state_dstate_stride", i64),
        ("x_batch_stride", i64), ("x_head_stride", i64), ("x_dim_stride", i64),
        ("dt_batch_stride", i64), ("dt_head_stride", i64), ("dt_dim_stride", i64),
        ("dt_bias_head_stride", i64), ("dt_bias_dim_stride", i64),
        ("A_head_stride", i64), ("A_dim_stride", i64), ("A_dstate_stride", i64),
        ("B_batch_stride", i64), ("B_group_stride", i64), ("B_dstate_stride", i64),
        ("C_batch_stride", i64), ("C_group_stride", i64), ("C_dstate_stride", i64),
        ("D_head_stride", i64), ("D_dim_stride", i64),
        ("z_batch_stride", i64), ("z_head_stride", i64), ("z_dim_stride", i64),
        ("out_batch_stride", i64), ("out_head_stride", i64), ("out_dim_stride", i64),
        ("state", vp), ("x", vp), ("dt", vp), ("dt_bias", vp), ("A_log", vp), ("B", vp), ("C", vp),
        ("D", vp), ("z", vp),
        ("x_scale", vp), ("dt_scale", vp), ("dt_bias_scale", vp), ("A_log_scale", vp),
        ("state_scale", vp), ("B_scale", vp), ("C_scale", vp), ("D_scale", vp), ("z_scale", vp),
        ("x_head_group_range", vp), ("x_dim_group_range", vp),
        ("out", vp),
    ]


class QaGemmW8A8Params(C.Structure):
    _fields_ = [
        ("m", i32), ("n", i32), ("k", i32), ("out_type", i32), ("round_mode", i32),
        ("a_scale_numel", i32), ("w_scale_numel", i32), ("use_alpha", i32),
        ("alpha", f32), ("scale_order", i32),
        ("lda", i64), ("ldw", i64), ("ldd", i64),
        ("a", vp), ("w", vp), ("a_scale", vp), ("w_scale", vp), ("d", vp),
    ]


class QaGemmW4A8Params(C.Structure):
    _fields_ = [
        ("m", i32), ("n", i32), ("k", i32), ("group_size", i32), ("out_type", i32),
        ("tok_scale_numel", i32), ("output_transpose", i32), ("reserved0", i32),
        ("lda", i64), ("ldd", i64),
        ("a", vp), ("w_packed", vp), ("s_group", vp), ("s_channel", vp), ("s_token", vp), ("d", vp),
        ("w8_workspace", vp), ("w8_workspace_bytes", i64),
    ]


class QaSsdParams(C.Structure):
    _fields_ = [
        ("batch", i32), ("seqlen", i32), ("nheads", i32), ("headdim", i32), ("dstate", i32),
        ("ngroups", i32), ("chunk_size", i32), ("dt_softplus", i32), ("dt_is_fp32", i32),
        ("D_has_hdim", i32), ("nhead_groups", i32), ("ndim_groups", i32),
        ("final_state_is_fp32", i32), ("reserved0", i32),
        ("dt_min", f32), ("dt_max", f32),
        ("x", vp), ("dt", vp), ("A_log", vp), ("B", vp), ("C", vp), ("D", vp), ("z", vp),
        ("dt_bias", vp),
        ("x_scale", vp), ("dt_scale", vp), ("A_log_scale", vp), ("B_scale", vp), ("C_scale", vp),
        ("D_scale", vp), ("z_scale", vp), ("state_scale", vp),
        ("x_head_group_range", vp), ("x_dim_group_range", vp),
        ("out", vp), ("final_states", vp), ("workspace", vp), ("workspace_bytes", i64),
    ]


# name -> (restype, argtypes); every symbol declared in include/quamba_amd.h
SYMBOLS = {
    "qa_status_string": (C.c_char_p, [C.c_int]),
    "qa_abi_version": (C.c_int, []),
    "qa_last_hip_error": (C.c_int, []),
    "qa_causal_conv1d_fwd": (C.c_int, [C.POINTER(QaConvParams), vp]),
    "qa_causal_conv1d_update": (C.c_int, [C.POINTER(QaConvParams), vp]),
    "qa_quamba2_conv1d_fwd": (C.c_int, [C.POINTER(QaConv2Params), vp]),
    "qa_quamba2_conv1d_update": (C.c_int, [C.POINTER(QaConv2Params), vp]),
    "qa_hadamard_quant": (C.c_int, [C.POINTER(QaHadamardParams), vp]),
    "qa_rmsnorm_gated": (C.c_int, [C.POINTER(QaNormGatedParams), vp]),
    "qa_rmsnorm_gated_hadamard_quant": (C.c_int, [C.POINTER(QaNormGatedParams), C.POINTER(QaHadamardParams), vp]),
    "qa_sscan_fwd": (C.c_int, [C.POINTER(QaSScanParams), vp]),
    "qa_sscan_chosen_mapping": (C.c_int, [C.POINTER(QaSScanParams)]),
    "qa_ssm_state_update": (C.c_int, [C.POINTER(QaSsmUpdateParams), vp]),
    "qa_mamba1_decode_step": (C.c_int, [C.POINTER(QaConvParams), C.POINTER(QaSsmUpdateParams), vp]),
    "qa_gemm_w8a8": (C.c_int, [C.POINTER(QaGemmW8A8Params), vp]),
    "qa_gemm_w4a8": (C.c_int, [C.POINTER(QaGemmW4A8Params), vp]),
    "qa_ssd_workspace_bytes": (C.c_int64, [C.POINTER(QaSsdParams)]),
    "qa_ssd_chunk_scan_fwd": (C.c_int, [C.POINTER(QaSsdParams), vp]),
    "qa_ssd_chunk_scan_fwd_noalloc": (C.c_int, [C.POINTER(QaSsdParams), vp]),
}

_lib = None


def lib():
    """Loads the shared library once; raises if it is not built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m quamba_amd.build` "
                "(quamba_amd has no CPU or PyTorch fallback)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.qa_abi_version() != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {handle.qa_abi_version()}, this binding expects "
                               f"{ABI_VERSION}: rebuild it with `python -m quamba_amd.build --force`")
        _lib = handle
    return _lib


def check(status, what):
    if status != QA_OK:
        l = lib()
        msg = l.qa_status_string(status).decode()
        extra = f" (hip error {l.qa_last_hip_error()})" if status == -5 else ""
        if status == -4:
            raise NotImplementedError(f"{what}: {msg}")
        raise RuntimeError(f"{what}: {msg}{extra}")


def ptr(t):
    """Device pointer of a torch tensor (or None)."""
    return None if t is None else t.data_ptr()


def current_stream(device):
    import torch
    return torch.cuda.current_stream(device).cuda_stream

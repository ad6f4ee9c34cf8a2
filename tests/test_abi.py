"""CPU-side checks of the C ABI: the library loads and exports every declared symbol, the ctypes
structs match the header's layout, and argument validation returns the documented codes."""
import ctypes as C
import os
import re
import subprocess

import pytest

from quamba_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "quamba_amd.h")


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qa_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = _declared_functions()
    assert len(names) >= 10
    assert sorted(_lib.SYMBOLS) == names
    handle = _lib.lib()
    for n in names:
        assert getattr(handle, n) is not None


def test_abi_version_and_status_strings():
    l = _lib.lib()
    assert l.qa_abi_version() == _lib.ABI_VERSION == 2
    assert l.qa_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5, -6):
        assert l.qa_status_string(code) not in (b"ok", b"unknown status")


def _param_structs():
    """Every parameter block the header declares, and its ctypes twin."""
    text = open(HEADER).read()
    names = sorted(set(re.findall(r"\}\s*(Qa[A-Za-z0-9]+Params)\s*;", text)))
    assert len(names) >= 9, names
    return [(n, getattr(_lib, n)) for n in names]


def _layout_from_gcc(tmp_path, structs):
    """sizeof and the offsetof of every field, as a C compiler lays the header's structs out."""
    lines = []
    for name, cls in structs:
        lines.append(f'printf("{name} . %zu\\n", sizeof({name}));')
        for field, _ in cls._fields_:
            lines.append(f'printf("{name} {field} %zu\\n", offsetof({name}, {field}));')
    src = tmp_path / "layout.c"
    src.write_text(f'#include <stddef.h>\n#include <stdio.h>\n#include "{HEADER}"\nint main(){{{"".join(lines)}return 0;}}\n')
    exe = tmp_path / "layout"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    return {(a, b): int(c) for a, b, c in (line.split() for line in out.strip().splitlines())}


def test_struct_layouts_match_the_header(tmp_path):
    """Size and the offset of every field of every Qa*Params block: a field of the binding that the header does not
    have fails to compile, a missing or reordered one moves an offset or the size."""
    structs = _param_structs()
    want = _layout_from_gcc(tmp_path, structs)
    for name, cls in structs:
        assert want[(name, ".")] == C.sizeof(cls), name
        for field, _ in cls._fields_:
            assert want[(name, field)] == getattr(cls, field).offset, f"{name}.{field}"
        # the header has no field the binding lacks: the fields tile the struct up to alignment padding
        covered = sum(C.sizeof(t) for _, t in cls._fields_)
        assert C.sizeof(cls) - covered < 8 * len(cls._fields_) and covered <= C.sizeof(cls), name


def test_a_swapped_pair_of_fields_is_caught(tmp_path):
    """The check above fails when two neighbouring fields of equal size change places in the binding."""
    class Swapped(C.Structure):
        _fields_ = [(n, t) for n, t in _lib.QaGemmW8A8Params._fields_]
    names = [n for n, _ in Swapped._fields_]
    i, j = names.index("lda"), names.index("ldw")

    class Swapped2(C.Structure):
        _fields_ = [f for f in Swapped._fields_[:i]] + [Swapped._fields_[j], Swapped._fields_[i]] + list(Swapped._fields_[j + 1:])
    want = _layout_from_gcc(tmp_path, [("QaGemmW8A8Params", _lib.QaGemmW8A8Params)])
    assert C.sizeof(Swapped2) == want[("QaGemmW8A8Params", ".")]
    assert any(want[("QaGemmW8A8Params", f)] != getattr(Swapped2, f).offset for f, _ in Swapped2._fields_)


def test_validation_codes_without_a_gpu():
    l = _lib.lib()
    assert l.qa_causal_conv1d_fwd(None, None) == -1
    p = _lib.QaConvParams()
    p.batch, p.dim, p.seqlen, p.width = 1, 8, 16, 4
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -1          # null pointers
    p.x = p.weight = p.out = 16                                     # never dereferenced on these paths
    p.width = 5
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -2          # width outside [2,4]
    p.width = 4
    p.x_l_stride, p.x_c_stride = 3, 5
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -3          # neither dimension contiguous
    p.seqlen = 0
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == 0           # empty input: nothing to launch
    x, p.x, p.out = p.x, 0, 0
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == 0           # tensors without elements may be null
    p.x = p.out = x
    p.seqlen, p.x_l_stride = 1, 1
    assert l.qa_causal_conv1d_update(C.byref(p), None) == -1       # conv_state missing
    p.conv_state = 16
    p.conv_state_len = 7
    assert l.qa_causal_conv1d_update(C.byref(p), None) == -2


def test_calls_over_no_elements_need_no_tensors():
    """Every entry point accepts null tensors when the sizes say there is nothing to read or write (an empty torch
    tensor has a null data pointer, and so has an empty std::vector), and returns before any HIP call."""
    l = _lib.lib()
    conv = _lib.QaConvParams()
    conv.dim, conv.seqlen, conv.width, conv.conv_state_len = 64, 16, 4, 4
    assert l.qa_causal_conv1d_fwd(C.byref(conv), None) == 0
    assert l.qa_causal_conv1d_update(C.byref(conv), None) == 0
    conv2 = _lib.QaConv2Params()
    conv2.dim, conv2.seqlen, conv2.width, conv2.x_dim, conv2.x_headdim, conv2.d_state, conv2.n_groups = 96, 16, 4, 64, 64, 16, 1
    conv2.xBC_c_stride = conv2.x_c_stride = conv2.B_c_stride = conv2.C_c_stride = 1
    conv2.conv_state_len = 4
    assert l.qa_quamba2_conv1d_fwd(C.byref(conv2), None) == 0
    assert l.qa_quamba2_conv1d_update(C.byref(conv2), None) == 0
    had = _lib.QaHadamardParams()
    had.dim = had.x_row_stride = had.out_row_stride = 5120
    assert l.qa_hadamard_quant(C.byref(had), None) == 0
    norm = _lib.QaNormGatedParams()
    norm.dim = norm.group_size = norm.x_row_stride = norm.out_row_stride = 256
    assert l.qa_rmsnorm_gated(C.byref(norm), None) == 0
    scan = _lib.QaSScanParams()
    scan.dim, scan.seqlen, scan.dstate, scan.n_groups = 64, 16, 16, 1
    assert l.qa_sscan_fwd(C.byref(scan), None) == 0
    upd = _lib.QaSsmUpdateParams()
    upd.nheads, upd.dim, upd.dstate, upd.ngroups = 1, 64, 16, 1
    assert l.qa_ssm_state_update(C.byref(upd), None) == 0
    assert l.qa_mamba1_decode_step(C.byref(conv), C.byref(upd), None) == 0
    for m, n in ((0, 64), (16, 0)):
        g8 = _lib.QaGemmW8A8Params()
        g8.m, g8.n, g8.k, g8.lda, g8.ldw, g8.ldd = m, n, 128, 128, 128, n
        g8.a_scale_numel = g8.w_scale_numel = 1
        assert l.qa_gemm_w8a8(C.byref(g8), None) == 0
        g4 = _lib.QaGemmW4A8Params()
        g4.m, g4.n, g4.k, g4.lda, g4.ldd, g4.group_size, g4.tok_scale_numel = m, n, 128, 128, n, 128, 1
        assert l.qa_gemm_w4a8(C.byref(g4), None) == 0
    ssd = _lib.QaSsdParams()
    ssd.seqlen, ssd.nheads, ssd.headdim, ssd.dstate, ssd.ngroups, ssd.chunk_size = 100, 4, 64, 128, 1, 64
    assert l.qa_ssd_chunk_scan_fwd(C.byref(ssd), None) == 0
    assert l.qa_ssd_chunk_scan_fwd_noalloc(C.byref(ssd), None) == 0
    # sizes that say there is something to do still need their tensors
    conv.batch, scan.batch, ssd.batch, had.rows = 1, 1, 1, 1
    assert l.qa_causal_conv1d_fwd(C.byref(conv), None) == -1
    assert l.qa_sscan_fwd(C.byref(scan), None) == -1
    assert l.qa_ssd_chunk_scan_fwd(C.byref(ssd), None) == -1
    assert l.qa_hadamard_quant(C.byref(had), None) == -1


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libquamba_amd.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()


def test_ssd_shape_limits_without_a_gpu():
    """qa_ssd_workspace_bytes validates the whole parameter block on the host: long problems whose launches are
    one-dimensional grids are accepted whatever the group count, a grid beyond 2^31 - 1 workgroups is refused."""
    l = _lib.lib()
    p = _lib.QaSsdParams()
    for f in ("x", "dt", "A_log", "B", "C", "out", "x_scale", "dt_scale", "A_log_scale", "B_scale", "C_scale"):
        setattr(p, f, 256)                                          # never dereferenced by the validation
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups, p.chunk_size = 16, 32768, 128, 64, 128, 8, 64
    assert l.qa_ssd_workspace_bytes(C.byref(p)) > 0                 # 16 x 512 chunks x 8 groups = 65536 (batch, chunk, group) triples
    p.batch, p.seqlen = 65536, 65536                                # 65536 x 1024 chunks x 128 heads > 2^31 - 1 workgroups
    assert l.qa_ssd_workspace_bytes(C.byref(p)) == 0
    assert l.qa_ssd_chunk_scan_fwd(C.byref(p), None) == -2
    p.batch, p.seqlen, p.dstate = 2, 512, 256                       # shapes the matrix-core kernels are not built for take the general ones
    assert l.qa_ssd_workspace_bytes(C.byref(p)) > 0
    p.headdim, p.chunk_size = 96, 100
    # 6 chunks: dt and the running sums in fp32 per (batch, head, chunk, step), entering states in fp16 per (batch, chunk, head,
    # channel, state), one x scale in fp32 and one row index of the state scales per (head, channel)
    assert l.qa_ssd_workspace_bytes(C.byref(p)) == 2 * (2 * 128 * 6 * 100 * 4) + 2 * 6 * 128 * 96 * 256 * 2 + 2 * 128 * 96 * 4
    for field, value in (("headdim", 257), ("dstate", 1025), ("chunk_size", 1025), ("chunk_size", 0)):
        q = _lib.QaSsdParams.from_buffer_copy(p)
        setattr(q, field, value)
        assert l.qa_ssd_chunk_scan_fwd(C.byref(q), None) == -4, field


def test_the_entry_point_without_allocation_refuses_large_problems_before_any_gpu_call():
    """The size check of qa_ssd_chunk_scan_fwd_noalloc comes before the first HIP call, so it can be checked here."""
    l = _lib.lib()
    p = _lib.QaSsdParams()
    for f in ("x", "dt", "A_log", "B", "C", "out", "x_scale", "A_log_scale", "B_scale", "C_scale"):
        setattr(p, f, 256)
    p.batch, p.seqlen, p.nheads, p.headdim, p.dstate, p.ngroups, p.chunk_size = 4, 4096, 80, 64, 128, 1, 256
    p.dt_is_fp32 = 1
    assert l.qa_ssd_workspace_bytes(C.byref(p)) > (64 << 20)
    assert l.qa_ssd_chunk_scan_fwd_noalloc(C.byref(p), None) == -6
    assert b"scratch" in l.qa_status_string(-6)


def test_scan_mapping_codes_without_a_gpu():
    """A mapping field without the marker bit of QA_SSCAN_MAPPING is refused before anything is launched, and
    qa_sscan_chosen_mapping reports the library's own choice (no GPU here: it assumes 256 CUs)."""
    from quamba_amd import ops
    l = _lib.lib()
    p = _lib.QaSScanParams()
    for f in ("u", "delta", "A_log", "B", "C", "out", "scale_u", "scale_delta", "scale_A", "scale_B", "scale_C"):
        setattr(p, f, 256)                                          # never dereferenced on these paths
    p.batch, p.dim, p.seqlen, p.dstate, p.n_groups = 8, 5120, 64, 16, 1
    for bad in (1, 0x10404, 0x40000000 | (3 << 28)):
        p.mapping = bad
        assert l.qa_sscan_fwd(C.byref(p), None) == -4, hex(bad)
    p.mapping = ops.sscan_mapping(3, 4)                             # well-formed, but no kernel has three lanes per channel
    assert l.qa_sscan_fwd(C.byref(p), None) == -4
    p.mapping = 0
    # 8 x 5120 channels on 1024 SIMDs: 2.5 four-lane waves per SIMD -> the last fifth of the channels takes eight lanes
    assert ops.sscan_chosen_mapping(8, 5120, 16) == (0, 64)
    assert ops.sscan_chosen_mapping(1, 5120, 16) == (8, 4)          # few waves: eight lanes per channel
    assert ops.sscan_chosen_mapping(4, 48, 16) == (4, 1)
    assert ops.sscan_chosen_mapping(8, 5120, 128) is None
    p.mapping = ops.sscan_mapping(4, 2)
    assert l.qa_sscan_chosen_mapping(C.byref(p)) == p.mapping       # a named mapping is reported as it is
    assert l.qa_sscan_chosen_mapping(None) == -1

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
    assert l.qa_abi_version() == 1
    assert l.qa_status_string(0) == b"ok"
    for code in (-1, -2, -3, -4, -5):
        assert l.qa_status_string(code) not in (b"ok", b"unknown status")


def test_struct_sizes_match_the_header(tmp_path):
    structs = ["QaConvParams", "QaSScanParams", "QaSsmUpdateParams", "QaGemmW8A8Params", "QaGemmW4A8Params",
               "QaSsdParams"]
    src = tmp_path / "sz.c"
    body = "".join(f'printf("{s} %zu\\n", sizeof({s}));' for s in structs)
    src.write_text(f'#include <stdio.h>\n#include "{HEADER}"\nint main(){{{body}return 0;}}\n')
    exe = tmp_path / "sz"
    subprocess.run(["gcc", str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    sizes = dict(line.split() for line in out.strip().splitlines())
    for s in structs:
        assert int(sizes[s]) == C.sizeof(getattr(_lib, s)), s


def test_validation_codes_without_a_gpu():
    l = _lib.lib()
    assert l.qa_causal_conv1d_fwd(None, None) == -1
    p = _lib.QaConvParams()
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -1          # null pointers
    p.x = p.weight = p.out = 16                                     # never dereferenced on these paths
    p.batch, p.dim, p.seqlen, p.width = 1, 8, 16, 5
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -2          # width outside [2,4]
    p.width = 4
    p.x_l_stride, p.x_c_stride = 3, 5
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == -3          # neither dimension contiguous
    p.seqlen = 0
    assert l.qa_causal_conv1d_fwd(C.byref(p), None) == 0           # empty input: nothing to launch
    p.seqlen, p.x_l_stride = 1, 1
    assert l.qa_causal_conv1d_update(C.byref(p), None) == -1       # conv_state missing
    p.conv_state = 16
    p.conv_state_len = 7
    assert l.qa_causal_conv1d_update(C.byref(p), None) == -2


def test_missing_library_fails_loudly(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libquamba_amd.so")
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        _lib.lib()

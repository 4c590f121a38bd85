"""CPU-side checks of the drop-in boundary: the shared library loads, exports every
symbol include/memorax_amd.h declares (and nothing is declared but missing), the Python
prototypes agree with the header's arity, and the host layer refuses non-GPU input
instead of falling back.  No kernel is launched."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "memorax_amd.h")


def _declared():
    src = open(HEADER).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    decls = {}
    for m in re.finditer(r"\b(mrx_\w+)\s*\(([^;{]*?)\)\s*;", src, flags=re.S):
        args = [a for a in m.group(2).split(",") if a.strip() and a.strip() != "void"]
        decls[m.group(1)] = len(args)
    return decls


def test_header_declares_the_expected_entry_points():
    names = set(_declared())
    assert {"mrx_linear_scan_fwd", "mrx_linear_scan_bwd", "mrx_linear_attn_fwd", "mrx_linear_attn_bwd",
            "mrx_delta_rule_fwd", "mrx_delta_rule_bwd", "mrx_chunk_size", "mrx_delta_chunk_size", "mrx_status_string",
            "mrx_version"} <= names


def test_library_exports_every_declared_symbol():
    from memorax_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build with memorax_amd/csrc/build.sh"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"


def test_python_prototypes_match_header_arity():
    from memorax_amd import _lib
    decl = _declared()
    assert set(_lib.SIGNATURES) == set(decl)
    for name, (_, args) in _lib.SIGNATURES.items():
        assert len(args) == decl[name], name


def test_status_strings_and_chunk_size_without_gpu():
    from memorax_amd import _lib
    lib = _lib.load()
    assert lib.mrx_status_string(0) == b"ok"
    assert b"unsupported" in lib.mrx_status_string(-2)
    assert lib.mrx_chunk_size(_lib.MRX_BF16) == 64 and lib.mrx_chunk_size(_lib.MRX_F32) == 32
    assert lib.mrx_delta_chunk_size(_lib.MRX_BF16) == 32 and lib.mrx_delta_chunk_size(_lib.MRX_F32) == 32
    assert lib.mrx_version() >= 100


def test_argument_validation_happens_before_any_launch():
    """Null pointers / bad sizes are rejected on the host (no GPU needed)."""
    from memorax_amd import _lib
    lib = _lib.load()
    n = None
    assert lib.mrx_linear_scan_fwd(n, n, n, n, n, n, n, n, n, 1, 1, 1, 0, 0, 0) == -1
    one = ctypes.c_void_p(16)
    assert lib.mrx_linear_scan_fwd(n, one, one, one, n, n, one, n, n, 0, 4, 4, 0, 0, 0) == -1
    assert lib.mrx_linear_scan_last(n, one, one, one, n, one, 2, 4, 4, 1, 1, 0) == -2  # bf16 final-state scan
    assert lib.mrx_mingru_scan_fwd(n, one, one, one, n, n, one, n, n, 2, 4, 4, 2, 0) == -2  # complex64 MinGRU
    assert lib.mrx_linear_scan_fwd(n, one, one, one, n, n, one, n, n, 2, 4, 4, 7, 0, 0) == -1  # no such dtype
    assert lib.mrx_linear_attn_fwd(n, one, one, one, one, n, one, n, n, 1, 8, 1, 72, 64, 1, 0, 0) == -2  # dk > 64
    assert lib.mrx_linear_attn_fwd(n, one, one, one, one, n, one, n, n, 1, 8, 1, 36, 64, 1, 0, 0) == -2  # 36 bf16: 4.5 segments
    assert lib.mrx_delta_rule_fwd(n, one, one, one, one, one, n, one, n, n, n, 1, 8, 1, 64, 72, 1, 0, 0, 0) == -2  # dv > 64
    assert lib.mrx_delta_rule_fwd(n, one, one, one, one, one, n, one, n, n, n, 1, 8, 1, 64, 64, 1, 0, 0, 3) == -1  # no such reset path
    assert lib.mrx_delta_rule_fwd_noalloc(n, one, one, one, one, one, n, one, n, 1, 8, 1, 32, 32, 1, 0) == -2  # 64 only
    assert lib.mrx_delta_rule_bwd(n, one, one, one, one, one, one, n, one, n, one, one, one, one, n,
                                  1, 8, 1, 64, 64, 0, 0, 0) == -1  # residual Tm_chk missing
    assert lib.mrx_linear_attn_bwd(n, one, one, one, one, one, n, one, n, one, one, one, n,
                                   1, 8, 1, 64, 64, 0, 0, 0) == -1  # S_last missing


def test_host_layer_has_no_cpu_fallback():
    from memorax_amd import kernels as K
    a = torch.rand(2, 4, 8)
    with pytest.raises(ValueError, match="GPU"):
        K.linear_scan_fwd(a, a.clone(), torch.zeros(2, 4, dtype=torch.bool))
    with pytest.raises(ValueError):
        K.linear_scan_fwd(a.double(), a.double(), torch.zeros(2, 4, dtype=torch.bool))


def test_missing_library_fails_loudly(monkeypatch):
    from memorax_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libmemorax_amd.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()

"""The C-ABI library loads and exports exactly what include/tybok_hip.h declares (no GPU needed)."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tybok_hip.h")


def _declared():
    text = open(HEADER, encoding="utf-8").read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tk_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_path():
    names = _declared()
    for required in ("tk_fp8w_gemm", "tk_fp8w_gated_ffn", "tk_expert_attn", "tk_pack_fp8_weight", "tk_last_error"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from tybok_amd import native

    if not os.path.exists(native.library_path()):
        pytest.skip("libtybok_hip.so not built (run python -m tybok_amd.csrc.build)")
    handle = ctypes.CDLL(native.library_path())
    for name in _declared():
        assert hasattr(handle, name), f"{name} declared in tybok_hip.h but not exported"
    # the ctypes table covers the header one to one
    assert sorted(native.SIGNATURES) == _declared()


def test_host_only_entry_points():
    from tybok_amd import native

    if not os.path.exists(native.library_path()):
        pytest.skip("libtybok_hip.so not built")
    lib = native.lib()
    assert lib.tk_version() >= 1
    assert lib.tk_fp8w_packed_bytes(2048, 720) == 64 * 23 * 1024  # K padded to 23 tiles of 32
    assert lib.tk_fp8w_packed_bytes(720, 2048) == 23 * 64 * 1024
    assert lib.tk_workspace_bytes() >= 32 << 20
    # argument validation happens on the host before any launch
    assert lib.tk_pack_fp8_weight(None, None, 32, 32, None) < 0
    assert b"bad argument" in lib.tk_last_error()


def test_missing_library_fails_loudly(monkeypatch):
    from tybok_amd import native

    monkeypatch.setattr(native, "_lib", None)
    monkeypatch.setattr(native, "_LIB_PATH", "/nonexistent/libtybok_hip.so")
    with pytest.raises(RuntimeError, match="no CPU or torch fallback"):
        native.lib()

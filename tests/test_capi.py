"""The C-ABI shared library loads without a GPU, exports every symbol the header
declares, and rejects bad arguments before touching the device."""

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "fouroversix_hip.h")


@pytest.fixture(scope="module")
def native():
    if not os.path.exists(os.path.join(ROOT, "fouroversix_amd", "libfouroversix_hip.so")):
        # (the build script by path: importing the package needs the libraries it builds)
        import importlib.util

        spec = importlib.util.spec_from_file_location("fos_build", os.path.join(ROOT, "fouroversix_amd", "build.py"))
        fos_build = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(fos_build)
        fos_build.build()
    from fouroversix_amd import _native

    return _native


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fos_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(native):
    L = native.lib()
    names = declared_functions()
    assert set(names) == set(native.EXPORTS)
    for name in names:
        assert getattr(L, name) is not None


def test_version_and_error_strings(native):
    L = native.lib()
    assert L.fos_version() >= 100
    assert L.fos_error_string(0) == b"success"
    for code in range(-6, 0):
        assert len(L.fos_error_string(code)) > 8
    assert b"unknown" in L.fos_error_string(-99)


def test_padding_and_workspace_queries(native):
    L = native.lib()
    assert (L.fos_padded_rows(1), L.fos_padded_rows(128), L.fos_padded_rows(129)) == (128, 128, 256)
    assert (L.fos_padded_cols(1), L.fos_padded_cols(64), L.fos_padded_cols(80)) == (64, 64, 128)
    assert L.fos_quantize_workspace_bytes(8192, 8192) >= 4


def test_argument_checks_need_no_device(native):
    """Every check below returns before the first HIP call."""
    L = native.lib()
    buf = ctypes.create_string_buffer(1 << 16)
    p = ctypes.addressof(buf)
    p = (p + 255) & ~255
    q = lambda **kw: L.fos_quantize(  # noqa: E731
        kw.get("x", p), kw.get("x_type", 0), kw.get("rows", 128), kw.get("cols", 64), kw.get("ld", 64),
        kw.get("dtype", 0), kw.get("rule", 3), kw.get("round", 0), 0, 0, 0, kw.get("layout", 1),
        kw.get("codes", p), kw.get("sf", p), kw.get("amax", p), 0, kw.get("ws", p), kw.get("ws_bytes", 1 << 15), None)
    assert q(x=None) == -4
    assert q(rows=0) == -1
    assert q(ld=32) == -1
    assert q(x_type=3) == -3
    assert q(x_type=2, x=p + 2) == -2  # fp32 elements: 4-byte aligned
    assert q(x_type=3, dtype=2, rule=0) == -3  # MXFP4: the same three element types
    assert q(x_type=2, dtype=2, rule=0, x=p + 2) == -2
    assert q(dtype=7) == -3
    assert q(rule=9) == -3
    assert q(dtype=1, rule=0) == -3  # IF4 has no static rule
    assert q(layout=5) == -3
    assert q(ws=None) == -5
    assert q(ws_bytes=8) == -5
    assert q(codes=p + 1) == -2
    g = lambda **kw: L.fos_gemm_nvfp4(  # noqa: E731
        kw.get("A", p), p, p, p, p, kw.get("M", 128), kw.get("N", 128), kw.get("K", 64), p, kw.get("out", 0),
        kw.get("ldd", 128), None, 0, None)
    assert g(A=None) == -4
    assert g(M=100) == -1  # fewer than 128 rows need K % 256 == 0
    assert L.fos_gemm_workspace_bytes(100, 128, 64) == 0
    assert L.fos_gemm_workspace_bytes(128, 1024, 8192) == 2 * 128 * 1024 * 4  # two splits of 16 K steps
    assert L.fos_gemm_workspace_bytes(128, 1024, 4096) == 0  # 16 steps: unsplit
    assert L.fos_gemm_workspace_bytes(8192, 8192, 8192) == 0
    assert g(K=32) == -1
    assert g(ldd=64) == -1
    assert g(out=2) == -3
    d = lambda **kw: L.fos_dequantize(  # noqa: E731
        kw.get("codes", p), p, p, kw.get("dtype", 0), 1, 1536.0, kw.get("rows", 128), 64,
        kw.get("rows_p", 128), 64, p, kw.get("out", 0), 64, kw.get("inter", 1), None)
    assert d(codes=None) == -4
    assert d(rows=200) == -1
    assert d(rows_p=100, rows=100) == -1
    assert d(dtype=3) == -3
    assert d(out=9) == -3
    assert d(inter=0) == -3  # value x scale meets in fp16 or fp32 only

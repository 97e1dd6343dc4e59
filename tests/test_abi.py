"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import ctypes
import os
import re

from ratchet_amd import _ffi

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "ratchet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"RT_API[^;(]*?\b(rt_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported():
    syms = header_symbols()
    assert len(syms) >= 20
    L = ctypes.CDLL(_ffi.LIB_PATH)
    missing = [s for s in syms if not hasattr(L, s)]
    assert not missing, missing
    assert sorted(_ffi.SIGNATURES) == syms  # the Python binding covers the same set


def test_rust_crate_declares_every_symbol():
    """crates/ratchet-hip-sys/src/lib.rs (source only: no rustc in the image) declares every symbol the header
    exports, with as many arguments, and nothing the header does not have."""
    text = open(os.path.join(ROOT, "include", "ratchet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    header = {m.group(1): m.group(2) for m in re.finditer(r"RT_API[^;(]*?\b(rt_[a-z0-9_]+)\s*\(([^;]*?)\)\s*;", text, flags=re.S)}
    rs = open(os.path.join(ROOT, "crates", "ratchet-hip-sys", "src", "lib.rs")).read()
    rs = re.sub(r"//[^\n]*", "", rs)
    rust = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (rt_[a-z0-9_]+)\s*\(([^;]*?)\)\s*(?:->[^;]*)?;", rs, flags=re.S)}
    assert sorted(rust) == sorted(header) == header_symbols()
    nargs = lambda a: 0 if a.strip() in ("", "void") else a.count(",") + 1
    for name in header:
        assert nargs(rust[name]) == nargs(header[name]), name
    # the structs the entry points take exist with the header's field counts
    for struct, fields in (("rt_matmul_desc", 13), ("rt_gemm_spec", 13), ("rt_attention_desc", 14),
                           ("rt_gguf_tensor_info", 6), ("rt_gguf_value", 7)):
        body = re.search(r"pub struct %s \{(.*?)\n\}" % struct, rs, flags=re.S).group(1)
        assert len(re.findall(r"pub \w+:", body)) == fields, struct


def test_status_and_kernel_strings():
    L = _ffi.lib()
    assert L.rt_status_string(_ffi.RT_OK) == b"RT_OK"
    assert L.rt_status_string(_ffi.RT_ERR_NO_DEVICE) == b"RT_ERR_NO_DEVICE"
    assert L.rt_kernel_string(_ffi.RT_KERNEL_GEMV_Q8) == b"gemv_q8"


def test_struct_layout_matches_header():
    # int32 x4, int64[8] x2, int32 x6, int64[8]  -> natural alignment, no surprises
    assert ctypes.sizeof(_ffi.MatmulDesc) == 16 + 128 + 24 + 64
    assert ctypes.sizeof(_ffi.GemmSpec) == 48 + 48 + 16


def test_no_device_is_a_status_not_a_crash():
    ctx = ctypes.c_void_p()
    st = _ffi.lib().rt_ctx_create(0, ctypes.byref(ctx))
    if st == _ffi.RT_OK:            # running on a GPU box
        assert ctx.value
        assert _ffi.lib().rt_ctx_destroy(ctx) == _ffi.RT_OK
        assert _ffi.lib().rt_ctx_create(10**6, ctypes.byref(ctx)) == _ffi.RT_ERR_NO_DEVICE
    else:
        assert st == _ffi.RT_ERR_NO_DEVICE and not ctx.value
    assert _ffi.lib().rt_ctx_create(0, None) == _ffi.RT_ERR_INVALID_ARG


def test_product_does_not_reference_the_oracle():
    """The shipped package must not import, load or link anything under oracle/."""
    pkg = os.path.join(ROOT, "ratchet_amd")
    for dirpath, _, files in os.walk(pkg):
        if "_build" in dirpath:
            continue
        for f in files:
            if f.endswith((".py", ".cpp", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src.lower(), os.path.join(dirpath, f)

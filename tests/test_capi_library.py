"""The C-ABI library loads without a GPU and exports every symbol include/esmoe.h declares."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "esmoe.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(esmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported(esmoe):
    from expert_specialization_moe_amd import _native

    names = _declared_functions()
    assert {"esmoe_fp8_blockwise_grouped_mm", "esmoe_mxfp8_grouped_mm", "esmoe_mxfp8_grouped_quant",
            "esmoe_gemm_workspace_bytes", "esmoe_last_error"} <= set(names)
    for name in names:
        assert hasattr(_native.lib, name), f"{name} declared in esmoe.h but not exported"


def test_argument_validation_needs_no_gpu(esmoe):
    from expert_specialization_moe_amd import _native

    lib = _native.lib
    assert lib.esmoe_gemm_workspace_bytes(32) >= 4 * (2 * 32 + 9)
    buf = (ctypes.c_char * 4096)()
    p = ctypes.cast(buf, ctypes.c_void_p)
    # k not a multiple of 128
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 4, 10, 128, 100, 0, p, 4096, None)
    assert rc == -1 and "k must be" in _native.last_error()
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 2000, 10, 128, 128, 0, p, 4096, None)
    assert rc == -1 and "num_experts" in _native.last_error()
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 4, 10, 128, 128, 48, p, 4096, None)
    assert rc == -1 and "force_bm" in _native.last_error()
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 4, 10, 128, 128, 0, p, 8, None)
    assert rc == -2 and "workspace" in _native.last_error()
    # a workspace that is not 16-byte aligned (the kernel reads its schedule records with 16-byte scalar loads)
    base = ctypes.addressof(buf)
    odd = ctypes.c_void_p(base + (16 - base % 16) % 16 + 4)
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 4, 10, 128, 128, 0, odd, 2048, None)
    assert rc == -1 and "16-byte aligned" in _native.last_error()
    rc = lib.esmoe_mxfp8_grouped_quant(p, 7, p, p, p, p, p, 4, 10, 128, 128, None)
    assert rc == -1 and "in_dtype" in _native.last_error()
    rc = lib.esmoe_mxfp8_grouped_quant(p, 0, p, p, p, p, p, 4, 10, 100, 128, None)
    assert rc == -1 and "sf_rows" in _native.last_error()
    # a size without a pointer is not the "library's own workspace" form (null pointer AND zero bytes)
    rc = lib.esmoe_fp8_blockwise_grouped_mm(p, 0, p, p, p, p, p, p, 4, 10, 128, 128, 0, None, 4096, None)
    assert rc == -2 and "workspace" in _native.last_error()
    header = open(os.path.join(ROOT, "include", "esmoe.h")).read()
    abi = int(re.search(r"#define ESMOE_ABI (\d+)", header).group(1))
    assert lib.esmoe_version() == f"esmoe 0.{abi} (gfx950)".encode()

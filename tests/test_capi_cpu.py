"""CPU-only checks of the drop-in boundary: libnvf_hip.so loads without a GPU, exports exactly the
entry points include/nvf_hip.h declares, and rejects bad arguments before touching the device."""
import ctypes
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nvf_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"NVF_API\s+[\w\s\*]+?\b(nvf_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_symbols()
    for required in ("nvf_nvfp4_block_quantize", "nvf_nvfp4_grouped_block_quantize", "nvf_nvfp4_scaled_mm",
                     "nvf_mxfp8_scaled_mm", "nvf_grouped_mm", "nvf_nvfp4_scaled_grouped_mm",
                     "nvf_preprocess_grouped_matmul_input_sf", "nvf_mxfp8_block_quantize", "nvf_nvfp4_scaled_mm_blockscale"):
        assert required in names
    assert len(names) >= 15


def test_library_loads_and_exports_every_declared_symbol():
    from fuser_amd import capi

    lib = capi.lib()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} is declared in nvf_hip.h but not exported"
        assert name in capi.SIGNATURES, f"{name} has no ctypes prototype in fuser_amd/capi.py"
    out = subprocess.run(["nm", "-D", "--defined-only", capi.LIB_PATH], capture_output=True, text=True, check=True).stdout
    exported = sorted(set(re.findall(r"\b(nvf_\w+)$", out, flags=re.M)))
    assert exported == declared_symbols(), "exported nvf_* symbols and the header disagree"


def test_header_compiles_as_plain_c():
    src = '#include "nvf_hip.h"\nint main(void) { return (int)NVF_OK; }\n'
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), "-x", "c", "-", "-fsyntax-only"],
                       input=src, text=True, capture_output=True)
    assert r.returncode == 0, r.stderr


def test_invalid_arguments_are_rejected_without_a_device():
    from fuser_amd import capi

    lib = capi.lib()
    p = ctypes.c_void_p(16)  # never dereferenced: every call below fails its checks first
    assert lib.nvf_nvfp4_block_quantize(p, capi.BF16, 4, 24, None, 1, p, p, None) == -2  # cols % 16
    assert b"block size 16" in lib.nvf_last_error()
    assert lib.nvf_nvfp4_block_quantize(p, 7, 4, 32, None, 1, p, p, None) == -1  # dtype
    assert lib.nvf_nvfp4_block_quantize(None, capi.BF16, 4, 32, None, 1, p, p, None) == -1  # NULL
    assert lib.nvf_nvfp4_block_quantize(None, capi.BF16, 0, 32, None, 1, None, None, None) == 0  # empty is a no-op
    assert lib.nvf_mxfp8_block_quantize(p, capi.BF16, 4, 48, 0, p, p, None) == -2
    assert lib.nvf_nvfp4_scaled_mm(p, p, p, p, p, p, 128, 128, 48, capi.BF16, None) == -2  # k % 32
    assert lib.nvf_nvfp4_scaled_mm(p, p, p, p, p, p, 128, 100, 64, capi.BF16, None) == -2  # n % 32
    assert lib.nvf_nvfp4_scaled_mm(p, p, p, p, p, p, 128, 128, 64, capi.F32, None) == -1  # out dtype
    assert lib.nvf_mxfp8_scaled_mm(p, p, p, p, p, p, 128, 128, 40, capi.BF16, None) == -2
    assert lib.nvf_nvfp4_scaled_mm_blockscale(p, p, p, p, p, p, p, p, p, 128, 128, 48, None) == -2  # k % 32
    assert lib.nvf_nvfp4_scaled_mm_blockscale(p, p, p, p, p, None, p, p, None, 128, 128, 64, None) == -1  # no global scale
    assert lib.nvf_nvfp4_scaled_mm_blockscale(None, None, None, None, None, None, None, None, None, 0, 128, 64, None) == 0
    assert lib.nvf_grouped_mm(p, p, p, p, p, 4, 128, 132, 64, capi.BF16, None) == -2  # n % 8
    assert lib.nvf_grouped_mm(p, p, p, p, p, 4, 128, 128, 64, capi.F32, None) == -1
    assert lib.nvf_nvfp4_scaled_grouped_mm(p, p, p, p, p, p, p, p, p, 4, 128, 128, 96, capi.BF16, None) == -2  # k % 64
    assert lib.nvf_nvfp4_scaled_grouped_mm(p, p, p, p, p, p, p, p, p, 2000, 128, 128, 128, capi.BF16, None) == -2  # groups
    q = ctypes.c_void_p(24)  # 8-byte aligned only: the GEMMs move 16-byte pieces
    assert lib.nvf_nvfp4_scaled_mm(q, p, p, p, p, p, 128, 128, 64, capi.BF16, None) == -1
    assert b"16-byte aligned" in lib.nvf_last_error()
    assert lib.nvf_mxfp8_scaled_mm(p, p, p, q, p, p, 128, 128, 64, capi.BF16, None) == -1
    assert lib.nvf_grouped_mm(p, p, q, p, p, 4, 128, 128, 64, capi.BF16, None) == -1
    assert lib.nvf_nvfp4_scaled_grouped_mm(p, q, p, p, p, p, p, p, p, 4, 128, 128, 128, capi.BF16, None) == -1
    assert lib.nvf_nvfp4_scaled_mm_blockscale(p, p, p, p, p, p, p, q, p, 128, 128, 64, None) == -1
    assert lib.nvf_preprocess_grouped_matmul_input_sf(p, 3, 4, 4, p, p, 1, p, None) == -1
    assert lib.nvf_status_string(-2) == b"unsupported shape"
    with pytest.raises(capi.NvfError):
        capi.check(-2)

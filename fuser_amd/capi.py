"""ctypes view of the C ABI declared in include/nvf_hip.h (raw device pointers in, status out)."""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libnvf_hip.so")

F32, BF16, F16 = 0, 1, 2
STATIC_SCRATCH_BYTES = 32 << 20  # NVF_STATIC_SCRATCH_BYTES

_p, _i64, _int = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int

SIGNATURES = {
    "nvf_status_string": (ctypes.c_char_p, [_int]),
    "nvf_last_error": (ctypes.c_char_p, []),
    "nvf_get_arch_version": (_int, [_p]),
    "nvf_get_multiprocessor_count": (_int, [_p]),
    "nvf_nvfp4_block_quantize": (_int, [_p, _int, _i64, _i64, _p, _int, _p, _p, _p]),
    "nvf_nvfp4_grouped_block_quantize": (_int, [_p, _int, _i64, _i64, _p, _p, _int, _p, _p, _p, _p]),
    "nvf_nvfp4_silu_mul_block_quantize": (_int, [_p, _p, _int, _i64, _i64, _p, _p, _int, _p, _p, _p, _p]),
    "nvf_nvfp4_global_scale": (_int, [_p, _int, _i64, _p, _p]),
    "nvf_preprocess_grouped_matmul_input_sf": (_int, [_p, _int, _i64, _i64, _p, _p, _int, _p, _p]),
    "nvf_mxfp8_block_quantize": (_int, [_p, _int, _i64, _i64, _int, _p, _p, _p]),
    "nvf_cast_f32_to_e2m1": (_int, [_p, _i64, _p, _p]),
    "nvf_cast_f32_to_e4m3": (_int, [_p, _i64, _p, _p]),
    "nvf_cast_f32_to_e8m0": (_int, [_p, _i64, _p, _p]),
    "nvf_nvfp4_scaled_mm": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p]),
    "nvf_nvfp4_scaled_mm_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "nvf_nvfp4_scaled_mm_ws": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p, _i64, _p]),
    "nvf_nvfp4_scaled_mm_static_ws": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p]),
    "nvf_nvfp4_scaled_mm_blockscale": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _p]),
    "nvf_mxfp8_scaled_mm": (_int, [_p, _p, _p, _p, _p, _p, _i64, _i64, _i64, _int, _p]),
    "nvf_grouped_mm": (_int, [_p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _int, _p]),
    "nvf_nvfp4_scaled_grouped_mm": (_int, [_p, _p, _p, _p, _p, _p, _p, _p, _p, _int, _i64, _i64, _i64, _int, _p]),
    "nvf_selftest_fast_division": (_int, [_p, _p]),
    "nvf_describe_dispatch": (_int, [ctypes.c_char_p, _i64, _i64, _i64, _int, _int, _i64, ctypes.c_char_p, _i64]),
}

_lib = None


def lib():
    """Loads libnvf_hip.so once and sets the prototypes; raises OSError when it is not built."""
    global _lib
    if _lib is None:
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def describe_dispatch(op, m, n, k, groups=1, dtype=BF16, workspace_bytes=0):
    """Kernels the GEMM entry point `op` would launch for this shape on a whole MI355X (no GPU needed)."""
    buf = ctypes.create_string_buffer(2048)
    check(lib().nvf_describe_dispatch(op.encode(), m, n, k, groups, dtype, workspace_bytes, buf, len(buf)))
    return buf.value.decode()


class NvfError(RuntimeError):
    pass


def check(status):
    if status != 0:
        l = lib()
        raise NvfError(f"{l.nvf_status_string(status).decode()}: {l.nvf_last_error().decode()}")

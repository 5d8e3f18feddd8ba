"""Python face of the CPU oracle.  TEST INFRASTRUCTURE ONLY.

Only tests, ``__graft_entry__.smoke`` and the ``cpu_baseline`` leg of ``bench.py`` may import
this module; the product (``fuser_amd``) never does.  It wraps ``libnvf_oracle.so`` (the C
restatement in ``nvf_oracle.c``) with ctypes and adds the torch-CPU "dequantize then fp32 matmul"
reference that the reference's own GEMM tests use
(tests/python/direct/test_cutlass_nvfp4_gemm.py:31-52, test_cutlass_mxfp8_gemm.py:23-34,77-89,
test_cutlass_gemm.py:68-70).
"""
import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libnvf_oracle.so")

F32, BF16, F16 = 0, 1, 2
_DT = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: F16}


def build():
    """Compile the C restatement (gcc, a second or two)."""
    subprocess.run(["make", "-s", "-B", "-C", _HERE, "libnvf_oracle.so"], check=True)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    c_p, c_i64, c_int, c_f = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
    sig = {
        "orc_swizzle_128x4_offset": (c_i64, [c_i64, c_i64, c_i64]),
        "orc_f32_to_e2m1_n": (None, [c_p, c_i64, c_p]),
        "orc_f32_to_e4m3_n": (None, [c_p, c_i64, c_p]),
        "orc_f32_to_e8m0_rp_n": (None, [c_p, c_i64, c_p]),
        "orc_e4m3_to_f32": (c_f, [ctypes.c_uint8]),
        "orc_e2m1_to_f32": (c_f, [ctypes.c_uint8]),
        "orc_e8m0_to_f32": (c_f, [ctypes.c_uint8]),
        "orc_block_quantize_nvfp4": (None, [c_p, c_int, c_i64, c_i64, c_p, c_int, c_p, c_p]),
        "orc_grouped_block_quantize_nvfp4": (None, [c_p, c_int, c_i64, c_i64, c_p, c_p, c_int, c_p, c_p, c_p]),
        "orc_preprocess_grouped_sf": (None, [c_p, c_int, c_i64, c_i64, c_p, c_p, c_int, c_p]),
        "orc_block_quantize_mxfp8": (None, [c_p, c_int, c_i64, c_i64, c_p, c_p]),
        "orc_dequantize_nvfp4": (None, [c_p, c_p, c_i64, c_i64, c_f, c_p]),
        "orc_dequantize_mxfp8": (None, [c_p, c_p, c_i64, c_i64, c_p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _load()
    return _lib


def round_up(x, y):
    return (x + y - 1) // y * y


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _cpu(t):
    assert t.device.type == "cpu", "the oracle runs on CPU tensors only"
    return t.contiguous()


# --------------------------------------------------------------------------- codecs
def f32_to_e2m1(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_f32_to_e2m1_n(x.ctypes.data, x.size, out.ctypes.data)
    return out


def f32_to_e4m3(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_f32_to_e4m3_n(x.ctypes.data, x.size, out.ctypes.data)
    return out


def f32_to_e8m0_rp(x: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_f32_to_e8m0_rp_n(x.ctypes.data, x.size, out.ctypes.data)
    return out


def e4m3_table() -> np.ndarray:
    return np.array([lib().orc_e4m3_to_f32(i) for i in range(256)], dtype=np.float32)


def e2m1_table() -> np.ndarray:
    return np.array([lib().orc_e2m1_to_f32(i) for i in range(16)], dtype=np.float32)


def e8m0_table() -> np.ndarray:
    return np.array([lib().orc_e8m0_to_f32(i) for i in range(256)], dtype=np.float32)


def swizzle_offset(row, col, padded_cols):
    return lib().orc_swizzle_128x4_offset(row, col, padded_cols)


# --------------------------------------------------------------------------- quantizers
def block_quantize_nvfp4(x: torch.Tensor, global_scale=None, swizzle=False):
    """-> (payload uint8 [M, K/2], scales uint8).  scales is [M, K/16] (linear) or
    [roundUp(M,128), roundUp(K/16,4)] (128x4 swizzle, padding bytes zero)."""
    x = _cpu(x)
    m, k = x.shape
    assert k % 16 == 0
    fp4 = torch.empty((m, k // 2), dtype=torch.uint8)
    if swizzle:
        sf = torch.zeros((round_up(m, 128), round_up(k // 16, 4)), dtype=torch.uint8)
    else:
        sf = torch.zeros((m, k // 16), dtype=torch.uint8)
    gs = None if global_scale is None else torch.tensor([float(global_scale)], dtype=torch.float32)
    lib().orc_block_quantize_nvfp4(_ptr(x), _DT[x.dtype], m, k, _ptr(gs), int(swizzle), _ptr(fp4), _ptr(sf))
    return fp4, sf


def grouped_block_quantize_nvfp4(x, input_offsets, output_offsets, global_scale=None, padded_rows=None):
    x = _cpu(x)
    m, k = x.shape
    io = _cpu(input_offsets).to(torch.int32)
    oo = _cpu(output_offsets).to(torch.int32)
    g = io.numel()
    if padded_rows is None:
        padded_rows = int(oo[-1]) + round_up(m - int(io[-1]), 128)
    fp4 = torch.empty((m, k // 2), dtype=torch.uint8)
    sf = torch.zeros((padded_rows, round_up(k // 16, 4)), dtype=torch.uint8)
    gs = None if global_scale is None else torch.tensor([float(global_scale)], dtype=torch.float32)
    lib().orc_grouped_block_quantize_nvfp4(
        _ptr(x), _DT[x.dtype], m, k, _ptr(io), _ptr(oo), g, _ptr(gs), _ptr(fp4), _ptr(sf)
    )
    return fp4, sf


def preprocess_grouped_sf(sf_linear, input_offsets, output_offsets, padded_rows=None):
    s = _cpu(sf_linear)
    m, c = s.shape
    io = _cpu(input_offsets).to(torch.int32)
    oo = _cpu(output_offsets).to(torch.int32)
    if padded_rows is None:
        padded_rows = int(oo[-1]) + round_up(m - int(io[-1]), 128)
    out = torch.zeros((padded_rows, round_up(c, 4)), dtype=s.dtype)
    lib().orc_preprocess_grouped_sf(_ptr(s), s.element_size(), m, c, _ptr(io), _ptr(oo), io.numel(), _ptr(out))
    return out


def block_quantize_mxfp8(x: torch.Tensor):
    """-> (e4m3 bytes [M, K], e8m0 bytes [M, K/32] linear)."""
    x = _cpu(x)
    m, k = x.shape
    assert k % 32 == 0
    q = torch.empty((m, k), dtype=torch.uint8)
    sf = torch.empty((m, k // 32), dtype=torch.uint8)
    lib().orc_block_quantize_mxfp8(_ptr(x), _DT[x.dtype], m, k, _ptr(q), _ptr(sf))
    return q, sf


# --------------------------------------------------------------------------- layout
def linear_to_swizzled_128_4(sf_linear: torch.Tensor) -> torch.Tensor:
    """Scatter by the index formula; padding bytes are zero."""
    s = _cpu(sf_linear)
    m, c = s.shape
    pc = round_up(c, 4)
    out = torch.zeros((round_up(m, 128) * pc,), dtype=s.dtype)
    r = torch.arange(m).view(-1, 1).expand(m, c)
    col = torch.arange(c).view(1, -1).expand(m, c)
    off = (r // 128) * pc * 128 + (col // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + col % 4
    out[off.reshape(-1)] = s.reshape(-1)
    return out.view(round_up(m, 128), pc)


def swizzled_to_linear_128_4(sf_swizzled: torch.Tensor, m, c) -> torch.Tensor:
    s = _cpu(sf_swizzled)
    pc = s.shape[1]
    r = torch.arange(m).view(-1, 1).expand(m, c)
    col = torch.arange(c).view(1, -1).expand(m, c)
    off = (r // 128) * pc * 128 + (col // 4) * 512 + (r % 32) * 16 + ((r % 128) // 32) * 4 + col % 4
    return s.reshape(-1)[off.reshape(-1)].view(m, c)


# --------------------------------------------------------------------------- dequantize + matmul
def dequantize_nvfp4(fp4_u8, sf_swizzled_u8, decode_scale=1.0) -> torch.Tensor:
    """Scalar C path (slow, small cases)."""
    a = _cpu(fp4_u8.view(torch.uint8))
    s = _cpu(sf_swizzled_u8.view(torch.uint8))
    m, kh = a.shape
    out = torch.empty((m, kh * 2), dtype=torch.float32)
    lib().orc_dequantize_nvfp4(_ptr(a), _ptr(s), m, kh * 2, float(decode_scale), _ptr(out))
    return out


def dequantize_mxfp8(fp8_u8, sf_swizzled_u8) -> torch.Tensor:
    a = _cpu(fp8_u8.view(torch.uint8))
    s = _cpu(sf_swizzled_u8.view(torch.uint8))
    m, k = a.shape
    out = torch.empty((m, k), dtype=torch.float32)
    lib().orc_dequantize_mxfp8(_ptr(a), _ptr(s), m, k, _ptr(out))
    return out


_E2M1 = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0])


def _unswizzle_fast(sf_u8, m, c):
    mp, cp = sf_u8.shape
    return sf_u8.reshape(mp // 128, cp // 4, 32, 4, 4).transpose(1, 3).reshape(mp, cp)[:m, :c]


def dequantize_nvfp4_fast(fp4_u8, sf_swizzled_u8, decode_scale=1.0) -> torch.Tensor:
    """Vectorised torch-CPU recipe: unpack nibbles -> LUT -> x un-swizzled e4m3 scale -> x decode scale
    (tests/python/direct_utils/narrow_precision.py:16-21,46-106)."""
    a = fp4_u8.view(torch.uint8)
    m, kh = a.shape
    k = kh * 2
    lo = (a & 0x0F).long()
    hi = (a >> 4).long()
    vals = torch.stack([_E2M1[lo], _E2M1[hi]], dim=-1).reshape(m, k)
    sf = _unswizzle_fast(sf_swizzled_u8.view(torch.uint8), m, k // 16).contiguous().view(torch.float8_e4m3fn).float()
    vals = (vals.view(m, k // 16, 16) * sf.unsqueeze(-1)).view(m, k)
    if decode_scale != 1.0:
        vals = vals * decode_scale
    return vals


def dequantize_mxfp8_fast(fp8_u8, sf_swizzled_u8) -> torch.Tensor:
    """fp8.float() * 2^(e8m0-127) (tests/python/direct/test_cutlass_mxfp8_gemm.py:23-34)."""
    a = fp8_u8.view(torch.uint8)
    m, k = a.shape
    sf = _unswizzle_fast(sf_swizzled_u8.view(torch.uint8), m, k // 32).contiguous()
    scale = torch.exp2(sf.float() - 127.0)
    vals = a.view(torch.float8_e4m3fn).float()
    return (vals.view(m, k // 32, 32) * scale.unsqueeze(-1)).view(m, k)


def ref_nvfp4_scaled_mm(a, b, sfa, sfb, alpha, fast=True) -> torch.Tensor:
    """fp32 result of alpha * dequant(a) @ dequant(b).T (cutlass/nvfp4_scaled_mm.cu:283-312 semantics)."""
    dq = dequantize_nvfp4_fast if fast else dequantize_nvfp4
    return torch.matmul(dq(a, sfa), dq(b, sfb).t()) * float(alpha)


def ref_nvfp4_scaled_mm_blockscale(a, b, sfa, sfb, alpha, global_normconst):
    """(payload [m, n/2] uint8, swizzled e4m3 scales) of the product quantized again along n, as the
    reference's own test states the expectation (tests/python/direct/test_cutlass_nvfp4_gemm.py:129-150:
    NVFP4-quantize the product with global scale global_normconst, scales to the 128x4 layout), applied to
    the fp32 product.  PARITY UNPINNED beyond that test's tolerances: the reference computes this in
    CUTLASS's LinCombBlockScaleFactor epilogue (cutlass/nvfp4_scaled_mm_blockscale.cu:87-93), a third-party
    header that is absent from the reference tree (empty submodule), so its exact rounding sequence
    (it is known to use an approximate reciprocal) cannot be restated here."""
    prod = ref_nvfp4_scaled_mm(a, b, sfa, sfb, alpha)
    return block_quantize_nvfp4(prod, float(global_normconst), True)


def ref_mxfp8_scaled_mm(a, b, sfa, sfb, alpha, fast=True) -> torch.Tensor:
    dq = dequantize_mxfp8_fast if fast else dequantize_mxfp8
    return torch.matmul(dq(a, sfa), dq(b, sfb).t()) * float(alpha)


def ref_grouped_mm(a, b, problem_sizes, expert_offsets) -> torch.Tensor:
    """Rows [off_e, off_e+m_e) of a times b[e].T in fp32 (cutlass/group_mm.cu:76-105 pointer rule).
    Rows owned by no group are returned as NaN so that a test can tell them apart."""
    m = a.shape[0]
    g, n, _ = b.shape
    out = torch.full((m, n), float("nan"), dtype=torch.float32)
    for e in range(g):
        off, me = int(expert_offsets[e]), int(problem_sizes[e][0])
        if me:
            out[off : off + me] = a[off : off + me].float() @ b[e].float().t()
    return out


def ref_nvfp4_scaled_grouped_mm(a, b, a_sf, b_sf, alphas, problem_sizes, expert_offsets, sf_offsets) -> torch.Tensor:
    """Per-expert NVFP4 GEMM (cutlass/nvfp4_scaled_group_mm.cu:83-155 pointer rule): expert e reads
    payload rows [off_e, off_e+m_e), scale rows [sf_off_e, sf_off_e+roundUp(m_e,128)), weight b[e]."""
    m = a.shape[0]
    g, n, kh = b.shape
    out = torch.full((m, n), float("nan"), dtype=torch.float32)
    a8, b8 = a.view(torch.uint8), b.view(torch.uint8)
    asf, bsf = a_sf.view(torch.uint8), b_sf.view(torch.uint8)
    for e in range(g):
        off, me, so = int(expert_offsets[e]), int(problem_sizes[e][0]), int(sf_offsets[e])
        if me == 0:
            continue
        da = dequantize_nvfp4_fast(a8[off : off + me], asf[so : so + round_up(me, 128)])
        db = dequantize_nvfp4_fast(b8[e], bsf[e])
        out[off : off + me] = (da @ db.t()) * float(alphas[e])
    return out


def compute_nvfp4_global_scale(tensor) -> float:
    """(448 * 6) / max|tensor| as a Python float that the caller stores as fp32; 1.0 for an all-zero tensor,
    clamped to the fp32 maximum (tests/python/direct/test_narrow_precision.py:138-156).  Pinned by closed
    forms in tests/test_oracle_fused_producers.py (amax 2688 -> 1, amax 1 -> 2688, zeros -> 1, tiny -> fp32 max)."""
    amax = torch.max(torch.abs(tensor)).to(torch.float32).item()
    if amax == 0.0:
        return 1.0
    return min(2688.0 / amax, torch.finfo(torch.float32).max)


def silu_mul(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``silu(gate) * up`` evaluated as the reference's layer does on bf16 / f16 tensors
    (benchmarks/python/layers_for_inference_benchmark.py:504): torch's silu, x / (1 + exp(-x)) in fp32 rounded
    to the tensor type, then the product in fp32 rounded to the tensor type.  Written out with explicit
    roundings so that it does not depend on the CPU's vectorised silu.  PARITY UNPINNED for the fused
    silu-mul quantizer built on it: the reference has no eager kernel or fixture for that fusion (its
    compiler generates one per graph); the GPU tests compare against this chain and against torch's own
    kernels on the GPU."""
    t = gate.dtype
    g = gate.float()
    act = (g / (1.0 + torch.exp(-g))).to(t)
    return (act.float() * up.float()).to(t)

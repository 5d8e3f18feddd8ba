"""Which kernel every BASELINE shape is dispatched to, pinned without a GPU through the dry run of
nvf_describe_dispatch (it walks the same launcher code as the real call and stops in front of each launch).
A tuning constant that silently reroutes one of the benchmark's shapes fails here."""
import pytest

from fuser_amd import capi

BF16, F16 = capi.BF16, capi.F16


def plan(op, m, n, k, groups=1, dtype=BF16, ws=0):
    return capi.describe_dispatch(op, m, n, k, groups, dtype, ws)


def test_config1_small_nvfp4_gemm_streams_the_weights():
    assert plan("nvfp4_scaled_mm", 256, 1024, 1024).startswith("nvfp4_skinny_ring_kernel<")


def test_config2_mxfp8_8192_cubed_takes_the_persistent_256x256_kernel():
    assert plan("mxfp8_scaled_mm", 8192, 8192, 8192) == "mxfp8_gemm_256_kernel<TM=4,stream_out=1> grid=256"
    assert plan("mxfp8_scaled_mm", 8192, 8192, 8192, dtype=F16) == "mxfp8_gemm_256_kernel<TM=4,stream_out=1> grid=256"


@pytest.mark.parametrize("m,n,k,kernel", [
    (16, 4096, 4096, "nvfp4_skinny_ring_kernel<RT=1,TT=1>"),
    (16, 14336, 4096, "nvfp4_skinny_ring_kernel<RT=4,TT=1>"),
    (16, 4096, 14336, "nvfp4_skinny_ring_kernel<RT=1,TT=1>"),
    (128, 4096, 4096, "nvfp4_skinny_ring_kernel<"),
    (128, 14336, 4096, "nvfp4_skinny_ring_kernel<"),
    (128, 4096, 14336, "nvfp4_skinny_ring_kernel<"),
    (2048, 4096, 4096, "nvfp4_gemm_256_kernel<grouped=0,TM=2,"),
    (2048, 14336, 4096, "nvfp4_gemm_256_kernel<grouped=0,TM=4,"),
    (2048, 4096, 14336, "nvfp4_gemm_256_kernel<grouped=0,TM=2,"),
])
def test_config3_llm_shapes(m, n, k, kernel):
    got = plan("nvfp4_scaled_mm", m, n, k)
    assert got.startswith(kernel) and ";" not in got, got


def test_config3_deep_k_with_a_workspace_splits_k():
    need = capi.lib().nvf_nvfp4_scaled_mm_workspace_bytes(128, 4096, 14336)
    assert need > 0
    assert plan("nvfp4_scaled_mm", 128, 4096, 14336, ws=need).startswith("nvfp4_tile_kernel<128,128,split_k>")
    assert plan("nvfp4_scaled_mm", 128, 4096, 14336, ws=need - 1).startswith("nvfp4_skinny_ring_kernel<")


def test_nvfp4_8192_cubed_takes_the_persistent_256x256_kernel():
    assert plan("nvfp4_scaled_mm", 8192, 8192, 8192).startswith("nvfp4_gemm_256_kernel<grouped=0,TM=4,f32=0,pairs=1> grid=256")


def test_config4_bf16_grouped_takes_the_persistent_kernel_in_one_launch():
    got = plan("grouped_mm", 8192, 14336, 4096, groups=8)
    assert got.startswith("grouped16_gemm_256_kernel<") and ";" not in got, got


@pytest.mark.parametrize("n,k", [(2048, 7168), (7168, 2048)])
def test_config5_nvfp4_grouped(n, k):
    got = plan("nvfp4_scaled_grouped_mm", 65536, n, k, groups=256)
    kernels = [g.split(" ")[0] for g in got.split("; ")]
    assert any(kk.startswith("nvfp4_gemm_256_kernel<grouped=1,TM=4") for kk in kernels), got  # the 256-row tiles of the large experts
    # the mid-sized experts: the kernel that converts their rows once per 512 weight rows (33-80 rows) and 128x256
    # tiles of the persistent kernel (81-128 rows and the ends of the large experts: no tile kernel)
    assert "nvfp4_group_panel_kernel<RT=4,TT=5,slots=2>" in got and "rows=33..80" in got, got
    assert any(kk.startswith("nvfp4_gemm_256_kernel<grouped=1,TM=2") for kk in kernels) and "rows=81..128 min_rows=129" in got, got
    assert "nvfp4_tile_kernel" not in got, got


def test_dry_run_reports_argument_errors_and_touches_no_device():
    buf = __import__("ctypes").create_string_buffer(64)
    assert capi.lib().nvf_describe_dispatch(b"mxfp8_scaled_mm", 128, 128, 40, 1, BF16, 0, buf, 64) == -2
    assert capi.lib().nvf_describe_dispatch(b"no_such_op", 128, 128, 64, 1, BF16, 0, buf, 64) == -1
    assert capi.lib().nvf_describe_dispatch(b"mxfp8_scaled_mm", 128, 128, 64, 1, BF16, 0, None, 64) == -1

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


def test_deep_k_with_a_workspace_splits_k_only_where_it_wins():
    lib = capi.lib()
    # config 3, M=128: the forms of the weight-streaming kernel without a split are as fast: no workspace asked for
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(128, 4096, 14336) == 0
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(128, 4096, 4096) == 0
    # one slab of 65..96 rows against N / 64 < compute units and 28+ chunks per split: K split over workgroups
    need = lib.nvf_nvfp4_scaled_mm_workspace_bytes(96, 4096, 14336)
    assert need == 4 * 96 * 4096 * 4
    got = plan("nvfp4_scaled_mm", 96, 4096, 14336, ws=need)
    assert got == "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=64x1x4 split_k + splitk_reduce_kernel", got
    got = plan("nvfp4_scaled_mm", 96, 4096, 14336, ws=need - 1)
    assert got.startswith("nvfp4_skinny_ring_kernel<") and "split_k" not in got, got
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(96, 4096, 4096) == 0
    # few tiles and a deep K: the streaming kernel where it runs (up to 256 rows, K % 32 == 0: a short last chunk is
    # fine), else the tile kernel's split
    for k in (8192, 8224):
        assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(128, 1024, k) == 0
        assert plan("nvfp4_scaled_mm", 128, 1024, k).startswith("nvfp4_skinny_ring_kernel<")
    need = lib.nvf_nvfp4_scaled_mm_workspace_bytes(384, 6176, 8224)
    assert need == 3 * 384 * 6176 * 4
    assert plan("nvfp4_scaled_mm", 384, 6176, 8224, ws=need).startswith("nvfp4_tile_kernel<128,128,split_k>")
    # (N no multiple of 256: the split only where it is estimated faster than streaming all columns or cutting them)
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(384, 4224, 8224) == 0
    assert plan("nvfp4_scaled_mm", 384, 4224, 8224) == "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=66x3"
    assert lib.nvf_nvfp4_scaled_mm_workspace_bytes(512, 4224, 8224) == 0
    assert plan("nvfp4_scaled_mm", 512, 4224, 8224) == "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=64x4; nvfp4_skinny_ring_kernel<RT=1,TT=2> grid=8x16"


@pytest.mark.parametrize("m,n,k,kernel", [
    (16, 4096, 4096, "mxfp8_skinny_kernel<RT=1,TT=1> grid=256x1"),
    (128, 4096, 4096, "mxfp8_skinny_kernel<RT=4,TT=2> grid=64x4"),
    (128, 14336, 4096, "mxfp8_skinny_kernel<RT=4,TT=4,W=4> grid=224x2"),
    (128, 4096, 14336, "mxfp8_skinny_kernel<RT=4,TT=2> grid=64x4"),
    (2048, 4096, 4096, "mxfp8_gemm_256_kernel<TM=2,stream_out=0> grid=256"),
    (2048, 14336, 4096, "mxfp8_gemm_256_kernel<TM=4,stream_out=0> grid=256"),
    # streaming or persistent kernel by estimated duration
    (256, 14336, 4096, "mxfp8_gemm_256_kernel<TM=2,stream_out=0> grid=112"),
    (256, 14336, 14336, "mxfp8_gemm_256_kernel<TM=2,stream_out=0> grid=112"),
    (512, 4096, 7168, "mxfp8_skinny_kernel<RT=4,TT=4,W=4> grid=64x8"),
    (512, 4096, 14336, "mxfp8_skinny_kernel<RT=4,TT=4> grid=64x8"),
    (1024, 2048, 14336, "mxfp8_skinny_kernel<RT=4,TT=4> grid=32x16"),
    (1024, 4096, 4096, "mxfp8_gemm_256_kernel<TM=2,stream_out=0> grid=128"),
    (1024, 8192, 4096, "mxfp8_gemm_256_kernel<TM=2,stream_out=0> grid=256"),
])
def test_mxfp8_llm_and_mid_sized_shapes(m, n, k, kernel):
    assert plan("mxfp8_scaled_mm", m, n, k).startswith(kernel), plan("mxfp8_scaled_mm", m, n, k)


def test_nvfp4_streaming_form_with_four_wavefronts_with_more_workgroups_than_compute_units():
    """128-row slabs x 64 weight rows, K % 128 == 0, more workgroups than the 256 compute units: workgroups of 4 wavefronts,
    two to a compute unit.  The form's measured gain is part of the streaming estimate among the streaming forms (160
    rows: two slabs of 128 rows instead of five of 32), and for 3072 <= K < 6144, by 4 %, against the persistent tiles."""
    four = "nvfp4_skinny_ring_kernel<RT=4,TT=8,W=4>"
    assert plan("nvfp4_scaled_mm", 256, 14336, 4096) == four + " grid=224x2"
    assert plan("nvfp4_scaled_mm", 160, 29568, 14336) == four + " grid=462x2"
    assert plan("nvfp4_scaled_mm", 160, 32896, 1024) == four + " grid=514x2"
    assert plan("nvfp4_scaled_mm", 1536, 12288, 4096) == four + " grid=192x12"
    assert plan("nvfp4_scaled_mm", 1536, 12288, 2048).startswith("nvfp4_gemm_256_kernel<grouped=0,TM=2")
    assert plan("nvfp4_scaled_mm", 128, 14336, 4096) == "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=224x1"
    assert plan("nvfp4_scaled_mm", 256, 14336, 2880) == "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=224x2"


def test_mxfp8_streaming_form_with_four_wavefronts_where_it_saves_a_round():
    """64-row x 64-column workgroups, more than the 256 compute units and at most twice as many: the form of which two
    share a compute unit (one round instead of two); otherwise, and with K % 128 != 0, the forms with 8 wavefronts."""
    four = "mxfp8_skinny_kernel<RT=4,TT=4,W=4>"
    assert plan("mxfp8_scaled_mm", 128, 14336, 4096) == four + " grid=224x2 m_base=0"
    assert plan("mxfp8_scaled_mm", 64, 28672, 4096) == four + " grid=448x1 m_base=0"
    assert plan("mxfp8_scaled_mm", 48, 28672, 4096) == four + " grid=448x1 m_base=0"
    assert plan("mxfp8_scaled_mm", 160, 7168, 2048) == four + " grid=112x3 m_base=0"
    assert plan("mxfp8_scaled_mm", 256, 8192, 2048) == four + " grid=128x4 m_base=0"
    for m, n, k in ((128, 7168, 2048), (256, 4096, 4096), (64, 16384, 8192), (128, 14336, 2880), (32, 28672, 4096)):
        got = plan("mxfp8_scaled_mm", m, n, k)
        assert got.startswith("mxfp8_skinny_kernel<") and "W=4" not in got, got
    assert "W=4" not in plan("mxfp8_scaled_mm", 320, 14336, 4096)


@pytest.mark.parametrize("m,n,k,kernel", [
    # streaming, persistent (256x256 / 128x256 tiles) or tile kernel by estimated duration
    (512, 4096, 4096, "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=64x4"),
    (1024, 2048, 4096, "nvfp4_skinny_ring_kernel<RT=4,TT=8> grid=32x8"),
    (640, 8192, 4096, "nvfp4_skinny_ring_kernel<RT=4,TT=8,W=4> grid=128x5"),
    (1024, 4096, 14336, "nvfp4_skinny_ring_kernel<RT=4,TT=8,W=4> grid=64x8"),
    (256, 14336, 4096, "nvfp4_skinny_ring_kernel<RT=4,TT=8,W=4> grid=224x2"),
    (1024, 8192, 4096, "nvfp4_gemm_256_kernel<grouped=0,TM=2,f32=0,pairs=1> grid=256"),
    (512, 14336, 4096, "nvfp4_gemm_256_kernel<grouped=0,TM=2,f32=0,pairs=1> grid=224"),
    (768, 14336, 4096, "nvfp4_gemm_256_kernel<grouped=0,TM=4,f32=0,pairs=1> grid=168"),
])
def test_nvfp4_mid_sized_shapes(m, n, k, kernel):
    assert plan("nvfp4_scaled_mm", m, n, k).startswith(kernel), plan("nvfp4_scaled_mm", m, n, k)


def test_nvfp4_dense_m_not_a_multiple_of_the_tile_height_takes_the_persistent_kernel_with_a_short_last_row_tile():
    op = "nvfp4_scaled_mm"
    # a prefill of any token count: one launch, the last row tile with fewer rows
    for m, n, k, tm, grid in ((4000, 4096, 4096, 4, 256), (8100, 8192, 8192, 4, 256), (384, 28672, 4096, 4, 224), (250, 28672, 4096, 2, 224)):
        got = plan(op, m, n, k)
        assert got.startswith(f"nvfp4_gemm_256_kernel<grouped=0,TM={tm},") and "ragged_m" in got and f"grid={grid} " in got and ";" not in got, (m, n, k, got)
    # where the weight-streaming kernel is estimated faster it takes all rows, and multiples of the tile height are as before
    got = plan(op, 1000, 4096, 14336)
    assert "skinny" in got and ";" not in got, got
    assert "ragged_m" not in plan(op, 4096, 4096, 4096) and "skinny" in plan(op, 300, 4096, 4096)
    # K % 128 != 0 has its own variant of the kernel: such a shape is still cut at a multiple of 128 rows
    got = plan(op, 4000, 4096, 2880).split("; ")
    assert len(got) == 2 and "ragged_k" in got[0] and "skinny" in got[1], got


def test_mxfp8_dense_m_not_a_multiple_of_the_tile_height_takes_the_persistent_kernel_with_a_short_last_row_tile():
    op = "mxfp8_scaled_mm"
    # a prefill of any token count: one launch, the last row tile with fewer rows
    for m, n, k, tm, grid in ((4000, 4096, 4096, 4, 256), (8100, 8192, 8192, 4, 256), (320, 14336, 4096, 2, 168), (640, 14336, 4096, 4, 168),
                              (96, 28672, 4096, 2, 112), (384, 28672, 4096, 4, 224)):
        got = plan(op, m, n, k)
        assert got.startswith(f"mxfp8_gemm_256_kernel<TM={tm},") and "ragged_m" in got and f"grid={grid}" in got and ";" not in got, (m, n, k, got)
    # where the weight-streaming kernel is estimated faster it takes all rows, and multiples of the tile height are as before
    got = plan(op, 1000, 4096, 14336)
    assert "skinny" in got and ";" not in got, got
    assert "ragged_m" not in plan(op, 4096, 4096, 4096) and "skinny" in plan(op, 300, 4096, 4096)
    # K % 128 != 0 as well: the variant with a short last K step and a short last row tile
    got = plan(op, 4000, 4096, 2880)
    assert got.startswith("mxfp8_gemm_256_kernel<TM=4,") and "ragged_k,ragged_m" in got and ";" not in got, got


@pytest.mark.parametrize("op", ["nvfp4_scaled_mm", "mxfp8_scaled_mm"])
def test_dense_n_not_a_multiple_of_256_is_cut_into_a_main_part_and_the_remaining_columns(op):
    got = plan(op, 8192, 29568, 8192).split("; ")
    assert len(got) == 2 and "gemm_256_kernel<" in got[0] and "TM=4" in got[0] and "grid=256" in got[0] and "skinny" in got[1], got
    # few rows: the weight-streaming kernel takes any N % 16 == 0 in one launch (MXFP8 from 65 rows on: one round of
    # 128x256 tiles with 100 rows each for the columns up to the last multiple of 256 is estimated faster)
    got = plan(op, 100 if op == "nvfp4_scaled_mm" else 48, 29568, 4096).split("; ")
    assert len(got) == 1 and "skinny" in got[0], got
    if op == "mxfp8_scaled_mm":
        got = plan(op, 100, 29568, 4096).split("; ")
        assert len(got) == 2 and got[0].startswith("mxfp8_gemm_256_kernel<TM=2,") and "ragged_m" in got[0] and "skinny" in got[1], got


def test_nvfp4_8192_cubed_takes_the_persistent_256x256_kernel():
    assert plan("nvfp4_scaled_mm", 8192, 8192, 8192).startswith("nvfp4_gemm_256_kernel<grouped=0,TM=4,f32=0,pairs=1> grid=256")


def test_config4_bf16_grouped_takes_the_persistent_kernel_in_one_launch():
    got = plan("grouped_mm", 8192, 14336, 4096, groups=8)
    assert got.startswith("grouped16_gemm_256_kernel<") and ";" not in got, got
    # from 128 rows per group on average, where its 256x256 tiles cover half the compute units; the tile kernels below
    assert plan("grouped_mm", 1024, 14336, 4096, groups=8).startswith("grouped16_gemm_256_kernel<")
    assert plan("grouped_mm", 8192, 2048, 7168, groups=64).startswith("grouped16_gemm_256_kernel<")
    assert plan("grouped_mm", 1000, 14336, 4096, groups=8).startswith("gemm16_kernel<")
    assert plan("grouped_mm", 1024, 4096, 14336, groups=8).startswith("gemm16_kernel<")  # 64 tiles of 256x256 only


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


@pytest.mark.parametrize("m,n,k,groups,streams,slots", [
    (512, 2048, 7168, 256, True, 15),     # a decode step: 64 tokens x top-8 (the benchmark's decode-sized call)
    (512, 7168, 2048, 256, True, 15),     # few rows in all: also against shallow weights
    (4096, 2048, 7168, 256, True, 124),   # a short prefill against deep weights
    (4096, 4096, 14336, 64, True, 64),
    (4096, 7168, 2048, 256, False, 0),    # shallow weights from 1025 rows on: 128x256 tiles of the persistent kernel
    (3072, 7168, 2048, 32, False, 0),     # 96 rows per group and one round of 256x256 tiles: no prefill yet
    (1536, 14336, 4096, 64, True, 46),
    (132, 2048, 7168, 256, True, 4),      # 128 workgroups: 8 wavefronts each
])
def test_nvfp4_grouped_below_the_prefill_size_streams_the_mid_sized_groups(m, n, k, groups, streams, slots):
    got = plan("nvfp4_scaled_grouped_mm", m, n, k, groups=groups)
    mid = [g for g in got.split("; ") if "rows=33..128" in g]
    assert len(mid) == 1, got
    if streams:
        # one block of N/64 workgroups per group that can exist with 33 rows or more, not one per expert
        # (more such workgroups than the 256 compute units: 4 wavefronts each, two to a compute unit)
        four = ",W=4" if slots * (n // 64) > 256 else ""
        assert mid[0].startswith(f"nvfp4_skinny_ring_kernel<RT=4,TT=8,grouped,nsplit=0{four}>") and f"grid={slots * (n // 64)} " in mid[0], got
    else:
        assert mid[0].startswith("nvfp4_gemm_256_kernel<grouped=1,TM=2"), got
    assert "nvfp4_group_panel_kernel" not in got, got


@pytest.mark.parametrize("m,n,k,groups,prefill", [
    (65536, 2048, 7168, 256, True), (6144, 2048, 7168, 256, True), (6000, 2048, 7168, 256, False),
    (1536, 14336, 4096, 8, True),     # a round of 256x256 tiles and 128 rows per group on average
    (2048, 14336, 4096, 64, False),   # a round, but 32 rows per group
    (3072, 14336, 4096, 64, True),    # two rounds
    (4096, 4096, 14336, 8, True), (3072, 4096, 14336, 8, False), (5632, 7168, 2048, 128, True), (4096, 7168, 2048, 256, False),
])
def test_nvfp4_grouped_counts_as_a_prefill_by_rows_or_by_rounds_of_256_row_tiles(m, n, k, groups, prefill):
    got = plan("nvfp4_scaled_grouped_mm", m, n, k, groups=groups)
    assert ("nvfp4_gemm_256_kernel<grouped=1,TM=4" in got) == prefill, got


def test_dry_run_reports_argument_errors_and_touches_no_device():
    buf = __import__("ctypes").create_string_buffer(64)
    assert capi.lib().nvf_describe_dispatch(b"mxfp8_scaled_mm", 128, 128, 40, 1, BF16, 0, buf, 64) == -2
    assert capi.lib().nvf_describe_dispatch(b"no_such_op", 128, 128, 64, 1, BF16, 0, buf, 64) == -1
    assert capi.lib().nvf_describe_dispatch(b"mxfp8_scaled_mm", 128, 128, 64, 1, BF16, 0, None, 64) == -1


@pytest.mark.parametrize("m", [1, 8, 32])
@pytest.mark.parametrize("n,k", [(2048, 7168), (7168, 2048), (256, 256), (512, 4096)])
def test_grouped_nvfp4_with_few_rows_in_all_launches_no_empty_grid(m, n, k):
    # a decode step of a few tokens x top-8: fewer rows in the whole call than the smallest group some launches serve
    got = plan("nvfp4_scaled_grouped_mm", m, n, k, groups=8)
    assert got and "grid=0" not in got, got


def test_blockscale_is_one_launch_and_ragged_shapes_add_only_the_fill_kernel():
    got = plan("nvfp4_scaled_mm_blockscale", 8192, 8192, 8192)
    assert got.startswith("nvfp4_gemm_256_kernel<") and "fp4_blockscale" in got and ";" not in got, got
    # (a call that streams whole zeroes the padding of the scale buffer in the same launch)
    ragged = plan("nvfp4_scaled_mm_blockscale", 200, 160, 512)
    assert ragged.startswith("nvfp4_skinny_ring_kernel<") and ";" not in ragged, ragged
    ragged = plan("nvfp4_scaled_mm_blockscale", 600, 160, 512).split("; ")
    assert len(ragged) == 2 and ragged[0].startswith("zero_fill_kernel") and ragged[1].startswith("nvfp4_tile_kernel<"), ragged
    # M no multiple of the tile height: one launch of the persistent kernel's variant with a short last row tile
    got = plan("nvfp4_scaled_mm_blockscale", 1000, 14336, 4096)
    assert got.startswith("nvfp4_gemm_256_kernel<grouped=0,TM=4,") and "fp4_blockscale,ragged_m" in got and ";" not in got, got
    # decode-sized calls stream the weights like the 16-bit op (one launch; the dump a second run of that kernel)
    got = plan("nvfp4_scaled_mm_blockscale", 128, 14336, 4096)
    assert got == plan("nvfp4_scaled_mm", 128, 14336, 4096) and got.startswith("nvfp4_skinny_ring_kernel<RT=4,TT=8>"), got
    dump = plan("nvfp4_scaled_mm_blockscale", 128, 14336, 4096, ws=4 * 128 * 14336).split("; ")
    assert len(dump) == 2 and dump[0] == dump[1], dump
    # the optional dump of the fp32 product is a second run of the same kernel
    dump = plan("nvfp4_scaled_mm_blockscale", 8192, 8192, 8192, ws=4 * 8192 * 8192).split("; ")
    assert len(dump) == 2 and "fp4_blockscale" in dump[0] and "f32=1" in dump[1], dump


KNOWN_KERNELS = ("nvfp4_skinny_ring_kernel<", "nvfp4_gemm_256_kernel<", "nvfp4_tile_kernel<", "nvfp4_group_panel_kernel<",
                 "gemm16_kernel<", "grouped16_gemm_256_kernel<", "mxfp8_gemm_256_kernel<", "mxfp8_skinny_kernel<", "mxfp8_gemm_kernel<",
                 "zero_fill_kernel", "nvfp4_act_convert_kernel", "nvfp4_skinny_f16a_kernel<", "splitk_reduce_kernel")


def _assert_known(got):
    assert got, "empty plan"
    assert "grid=0" not in got, got
    for part in got.split("; "):
        assert any(k in part for k in KNOWN_KERNELS), got


def test_sweep_of_other_shapes_reaches_a_kernel_on_every_branch():
    """Shapes off the benchmark's list: the dry run must return NVF_OK and name known kernels with non-empty grids,
    whatever the tuning constants of the dispatch are (catches dead or broken branches after a constant changes)."""
    ms = [1, 16, 17, 48, 100, 128, 129, 256, 300, 512, 1000, 2048, 4096, 8192]
    nks = [(32, 32), (64, 128), (128, 512), (256, 256), (512, 1024), (1024, 8192), (1536, 7168), (2048, 2048), (3072, 2048),
           (4096, 4096), (4128, 4096), (6144, 512), (7168, 2048), (14336, 4096), (28672, 4096), (4096, 14336), (256, 16384)]
    for m in ms:
        for n, k in nks:
            for ws in (0, 64 << 20):
                _assert_known(plan("nvfp4_scaled_mm", m, n, k, ws=ws))
            _assert_known(plan("nvfp4_scaled_mm_blockscale", m, n, k))
            _assert_known(plan("mxfp8_scaled_mm", m, n, k))
            _assert_known(plan("mxfp8_scaled_mm", m, n, k, dtype=F16))
            _assert_known(plan("grouped_mm", m, n, k, groups=1))
            for groups in (3, 8, 64, 256):
                _assert_known(plan("grouped_mm", m, n, k, groups=groups))
                if n % 128 == 0 and k % 64 == 0:
                    _assert_known(plan("nvfp4_scaled_grouped_mm", m, n, k, groups=groups))

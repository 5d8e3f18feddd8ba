"""Pins the oracle's narrow-float codecs (oracle/nvf_oracle.c) against golden tables, closed forms,
torch's own casts and the tie list of cvt.rn.satfinite (runtime/casts.cu:696-802, :911-1111)."""
import numpy as np
import torch

from helpers import all_bf16_as_f32, golden
from oracle import nvf_oracle as O


def test_e2m1_decode_table():
    # tests/python/direct_utils/narrow_precision.py:53-73
    expect = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]
    tab = O.e2m1_table()
    assert tab.tolist() == expect
    assert np.signbit(tab[8])


def test_e2m1_encode_all_bf16_against_golden():
    vals = all_bf16_as_f32()
    gold = golden("e2m1_of_bf16.npy")
    ok = ~np.isnan(vals)
    assert np.array_equal(O.f32_to_e2m1(vals[ok]), gold[ok])


def test_e2m1_ties_go_to_even_code_and_saturate():
    ties = np.array([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0], dtype=np.float32)
    assert O.f32_to_e2m1(ties).tolist() == [0, 2, 2, 4, 4, 6, 6]       # 0, 1, 1, 2, 2, 4, 4
    assert O.f32_to_e2m1(-ties).tolist() == [8, 10, 10, 12, 12, 14, 14]
    up = np.nextafter(ties, np.float32(np.inf))
    dn = np.nextafter(ties, np.float32(0))
    assert O.f32_to_e2m1(up).tolist() == [1, 2, 3, 4, 5, 6, 7]
    assert O.f32_to_e2m1(dn).tolist() == [0, 1, 2, 3, 4, 5, 6]
    big = np.array([6.0, 6.5, 1e30, np.inf, -7.0, -np.inf], dtype=np.float32)
    assert O.f32_to_e2m1(big).tolist() == [7, 7, 7, 7, 15, 15]
    assert O.f32_to_e2m1(np.array([0.0, -0.0], dtype=np.float32)).tolist() == [0, 8]


def test_e2m1_is_nearest_grid_point_on_random_fp32():
    rng = np.random.default_rng(0)
    x = (rng.standard_normal(1 << 18) * 3).astype(np.float32)
    code = O.f32_to_e2m1(x)
    grid = np.array([0, 0.5, 1, 1.5, 2, 3, 4, 6], dtype=np.float64)
    got = grid[code & 7]
    a = np.minimum(np.abs(x.astype(np.float64)), 6.0)
    best = np.min(np.abs(a[:, None] - grid[None, :]), axis=1)
    assert np.all(np.abs(got - a) == best)
    assert np.array_equal((code >> 3).astype(bool), np.signbit(x))
    # idempotent on the grid
    assert O.f32_to_e2m1(grid.astype(np.float32)).tolist() == list(range(8))


def test_e4m3_decode_matches_torch_for_all_codes():
    tab = O.e4m3_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(tab), np.isnan(ref))
    assert np.array_equal(tab[~np.isnan(tab)], ref[~np.isnan(ref)])


def test_e4m3_encode_all_bf16_against_golden_and_saturation():
    vals = all_bf16_as_f32()
    gold = golden("e4m3_of_bf16.npy")
    ok = ~np.isnan(vals)
    assert np.array_equal(O.f32_to_e4m3(vals[ok]), gold[ok])
    sat = np.array([448.0, 449.0, 463.9, 464.0, 1e9, np.inf, -1e9, -np.inf], dtype=np.float32)
    assert O.f32_to_e4m3(sat).tolist() == [0x7E] * 6 + [0xFE] * 2


def test_e4m3_encode_random_fp32_matches_torch_cast():
    rng = np.random.default_rng(1)
    x = (rng.standard_normal(1 << 18) * np.exp(rng.uniform(-14, 7, 1 << 18))).astype(np.float32)
    ref = torch.from_numpy(np.clip(x, -448, 448)).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    assert np.array_equal(O.f32_to_e4m3(x), ref)
    # round trip: every non-NaN code decodes and re-encodes to itself
    tab = O.e4m3_table()
    codes = np.array([c for c in range(256) if not np.isnan(tab[c])], dtype=np.uint8)
    assert np.array_equal(O.f32_to_e4m3(tab[codes]), codes)


def test_e8m0_round_up_is_ceil_log2():
    rng = np.random.default_rng(2)
    x = np.exp(rng.uniform(-80, 80, 1 << 16)).astype(np.float32)
    expect = np.clip(np.ceil(np.log2(x.astype(np.float64))) + 127, 0, 254).astype(np.uint8)
    assert np.array_equal(O.f32_to_e8m0_rp(x), expect)
    exact = np.array([1.0, 2.0, 0.5, 2.0**-127, 2.0**127], dtype=np.float32)
    assert O.f32_to_e8m0_rp(exact).tolist() == [127, 128, 126, 0, 254]
    just_above = np.nextafter(exact[:3], np.float32(np.inf))
    assert O.f32_to_e8m0_rp(just_above).tolist() == [128, 129, 127]
    assert O.f32_to_e8m0_rp(np.array([0.0, np.inf, 3e38], dtype=np.float32)).tolist() == [0, 254, 254]
    tab = O.e8m0_table()
    ref = torch.arange(255, dtype=torch.uint8).view(torch.float8_e8m0fnu).float().numpy()
    assert np.array_equal(tab[:255], ref) and np.isnan(tab[255])

"""The NVFP4 quantizer evaluates amax / 6 (runtime/block_quantization_kernels.cu:224) as a multiplication by
RN(1/6) plus one fused correction step.  tests/cpp/div6_check.c compares that form with the correctly rounded
quotient for EVERY fp32 value with biased exponent in [2, 250] -- the operands the kernel uses it for -- and
shows where it stops being exact (exponent 1: the residual's own rounding).  The reciprocal 1/x of the same
kernel depends on the GPU's v_rcp_f32 and is checked on the device (tests/test_gpu_codecs_quantize.py)."""
import os
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    exe = str(tmp_path_factory.mktemp("div6") / "div6_check")
    r = subprocess.run(["gcc", "-O2", "-march=native", "-ffp-contract=off", "-fno-fast-math",
                        os.path.join(ROOT, "tests", "cpp", "div6_check.c"), "-o", exe, "-lm"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    return exe


def test_div6_by_reciprocal_is_the_ieee_quotient_for_every_operand_the_kernel_uses(checker):
    # 249 exponents x 2^23 mantissas = 2.09e9 operands, split over the cores
    bounds = [(2, 32), (33, 64), (65, 96), (97, 128), (129, 160), (161, 192), (193, 224), (225, 250)]
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as pool:
        outs = list(pool.map(lambda b: subprocess.run([checker, str(b[0]), str(b[1])], capture_output=True, text=True, timeout=900), bounds))
    for b, r in zip(bounds, outs):
        assert r.returncode == 0 and r.stdout.startswith("mismatches 0 "), (b, r.stdout, r.stderr)


def test_div6_check_can_fail(checker):
    """The same program over the denormal results (biased exponent 0 and 1 of the operand): the form is not exact
    there, which is why the kernel excludes them -- and shows that the check above is able to find a mismatch."""
    r = subprocess.run([checker, "0", "1"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 1 and not r.stdout.startswith("mismatches 0 "), r.stdout

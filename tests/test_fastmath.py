"""Host checks of the arithmetic shortcuts the kernels rely on.

* div_by_invariant (aimet_amd/csrc/miq_fastmath.h) must equal IEEE binary32 division bit for bit inside its
  contract: the header is compiled for the host and compared with `/` on hundreds of millions of operand pairs.
* the multiply-high division by a launch-invariant 31-bit divisor (miq_common.h) must equal integer division.
* round_half_away (miq_fastmath.h), the three-operation roundf, must equal roundf for every float.
"""
import os
import subprocess

import numpy as np

from conftest import ROOT


def test_div_by_invariant_equals_ieee_division(tmp_path):
    exe = tmp_path / "fastdiv_check"
    src = os.path.join(ROOT, "tests", "host", "fastdiv_check.cpp")
    flags = ["-O2", "-std=c++17", "-ffp-contract=off"]
    if "fma" in open("/proc/cpuinfo").read():
        flags.append("-mfma")          # hardware fused multiply-add; otherwise libm's (slower, equally exact)
    subprocess.run(["g++", *flags, "-o", str(exe), src], check=True)
    out = subprocess.run([str(exe), "20"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:]
    assert out.stdout.startswith("OK")


def test_round_half_away_equals_roundf(tmp_path):
    exe = tmp_path / "round_check"
    src = os.path.join(ROOT, "tests", "host", "round_check.cpp")
    subprocess.run(["g++", "-O2", "-std=c++17", "-ffp-contract=off", "-o", str(exe), src], check=True)
    # every 5th bit pattern up to 2^24 in both signs + a dense sweep around the half-integers (about 10 s; stride 1
    # is the exhaustive walk)
    out = subprocess.run([str(exe), "5"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:]
    assert out.stdout.startswith("OK")


def _magic(d):
    s = 0
    while (1 << s) < d:
        s += 1
    return ((1 << (31 + s)) // d + 1) & 0xFFFFFFFF, s - 1


def test_multiply_high_division():
    rng = np.random.default_rng(0)
    divisors = [2, 3, 4, 5, 7, 9, 16, 17, 255, 256, 1000, 4096, 4608, 11008, 65535, 65536, 65537, (1 << 30) - 1,
                1 << 30, (1 << 31) - 1] + [int(v) for v in rng.integers(2, 1 << 31, 200)]
    for d in divisors:
        magic, shift = _magic(d)
        assert magic < (1 << 32)
        n = np.concatenate([rng.integers(0, 1 << 31, 20000, dtype=np.uint64),
                            np.array([0, 1, d - 1, d, d + 1, 2 * d - 1, 2 * d, (1 << 31) - 1], dtype=np.uint64),
                            (np.arange(1, 2000, dtype=np.uint64) * d) % (1 << 31),
                            (np.arange(1, 2000, dtype=np.uint64) * d - 1) % (1 << 31)])
        n = n[n < (1 << 31)]             # the dividend has at most 31 bits (the launcher guarantees it)
        q = ((n * np.uint64(magic)) >> np.uint64(32)) >> np.uint64(shift)
        assert np.array_equal(q, n // np.uint64(d)), d


def test_bucket_row_equals_the_reference_sequence(tmp_path):
    """bucket_row (miq_fastmath.h) answers most samples with one fused multiply-add and falls back to the reference's
    divide / subtract / round sequence near bucket edges; it must select the reference's bucket for every sample:
    thousands of PDF ranges over 60 decades, the floats around every bucket edge, random samples, arbitrary bit
    patterns."""
    exe = tmp_path / "bucket_check"
    src = os.path.join(ROOT, "tests", "host", "bucket_check.cpp")
    flags = ["-O2", "-std=c++17", "-ffp-contract=off"]
    if "fma" in open("/proc/cpuinfo").read():
        flags.append("-mfma")
    subprocess.run(["g++", *flags, "-o", str(exe), src], check=True)
    out = subprocess.run([str(exe), "3000"], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout[-2000:]
    assert out.stdout.startswith("OK")
    assert float(out.stdout.split()[2]) > 0.2          # the one-operation path did answer a good share

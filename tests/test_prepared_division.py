"""The short division sequence of the kernels (x * (r + rl) followed by one FMA correction, include/fk/exec/kernels.h)
against the host's IEEE division, exhaustively over the significands of x for a set of divisors.  CPU only: the same
float operations (fmaf) give the same bits on the host as on the GPU; the GPU side is covered by case 12 of
tests/cpp/api_gpu.cpp, which divides random, subnormal, infinite and zero operands on the device."""
import os
import subprocess

import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def test_short_division_is_correctly_rounded(tmp_path):
    src = os.path.join(HERE, "cpp", "prepared_division_check.c")
    exe = str(tmp_path / "prepared_division_check")
    flags = ["-O2", "-ffp-contract=off", "-fopenmp"]
    cpuinfo = open("/proc/cpuinfo").read() if os.path.exists("/proc/cpuinfo") else ""
    if " fma" in cpuinfo:
        flags.append("-mfma")  # fmaf as one instruction; without it the library routine gives the same values, slowly
        divisors = "48"
    else:
        divisors = "6"
    subprocess.run(["gcc", *flags, src, "-o", exe, "-lm"], check=True)
    res = subprocess.run([exe, divisors], capture_output=True, text=True, timeout=600)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "mismatches 0" in res.stdout

"""The fp8 quantizers replace x / s by a reciprocal and a residual correction (ksanallm_amd/csrc/fp8_quant.hip): the
host program tests/cpp/exact_div_test.c checks that sequence against the IEEE division over every scale mantissa."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reciprocal_with_residual_correction_is_the_ieee_quotient(tmp_path):
    with open("/proc/cpuinfo") as f:
        if " fma" not in f.read():
            pytest.skip("no hardware fma on this host: the exhaustive loop would take minutes in software")
    exe = str(tmp_path / "exact_div_test")
    subprocess.run(["gcc", "-O2", "-mfma", "-fopenmp", "-ffp-contract=off", os.path.join(ROOT, "tests", "cpp", "exact_div_test.c"),
                    "-o", exe, "-lm"], check=True)
    out = subprocess.run([exe], capture_output=True, text=True, timeout=600)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.count(" 0 mismatches") == 3, out.stdout

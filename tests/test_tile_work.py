"""Host check of the MFMA tile kernels' work order (csrc/tile_work.h), compiled with g++ and run on the CPU."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_every_tile_part_taken_once(tmp_path):
    exe = str(tmp_path / "tile_work_test")
    subprocess.run(["g++", "-O1", "-std=c++17", "-D__host__=", "-D__device__=", "-D__forceinline__=inline",
                    "-I" + os.path.join(ROOT, "ksanallm_amd", "csrc"), os.path.join(ROOT, "tests", "cpp", "tile_work_test.cpp"),
                    "-o", exe], check=True)
    out = subprocess.run([exe], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert out.stdout.startswith("OK")

"""The box of live k-slabs that the convolution kernel computes per tile (padding taps outside it are
never loaded) must contain every product whose tap lies inside the image.  The kernel's own index
functions are host-callable, so this is checked by brute force on the CPU: tests/slab_box_check.hip
includes csrc/conv_igemm.inc, is compiled for the host only and run."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_slab_box_contains_every_live_product(tmp_path):
    hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(hipcc):
        pytest.skip("hipcc not found")
    exe = str(tmp_path / "slab_box_check")
    subprocess.run([hipcc, "--cuda-host-only", "-O1", "-std=c++17", "-Wno-unused-function",
                    "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(ROOT, "dcgan-cuda_amd", "csrc"),
                    "-o", exe, os.path.join(ROOT, "tests", "slab_box_check.hip")], check=True)
    res = subprocess.run([exe], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout + res.stderr
    assert " 0 failures" in res.stdout, res.stdout

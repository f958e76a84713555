"""The kernel-table seam against the reference's own record, without a GPU: the table half of the host
library compiles unchanged against the reference's src/runtime/node.hh, this build's rt::Node has the
reference's layout field for field, and the HIP table has an entry wherever the reference's GPU table
has one on the convolution path (src/gpu/kernels.cu:23-61)."""
import ctypes as C
import os
import subprocess

import pytest

import seam

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
REF = "/root/reference"


def test_table_half_compiles_against_the_reference_header():
    if not os.path.isdir(os.path.join(REF, "src", "runtime")):
        pytest.skip("reference tree absent")
    host = os.path.join(ROOT, "dcgan-cuda_amd", "host")
    res = subprocess.run(["g++", "-std=c++14", "-fsyntax-only", "-Wall", "-M", "-I" + os.path.join(REF, "src", "runtime"),
                          "-I" + os.path.join(ROOT, "include"), "-I" + host, os.path.join(host, "hip_table.cc")],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    deps = res.stdout.replace("\\\n", " ").split()
    assert os.path.join(REF, "src", "runtime", "node.hh") in deps
    assert os.path.join(host, "node.hh") not in deps      # whose rt::Node it was compiled for


def test_node_layout_is_the_reference_one():
    if not seam.have():
        pytest.skip("oracle/_ref/libseam_ref.so not built (reference tree absent)")
    import __graft_entry__ as ge
    host = ge.load_package().hostabi.load()
    host.dg_node_layout.argtypes = [C.POINTER(C.c_ulong), C.c_int]
    mine, theirs = seam.layout(host.dg_node_layout), seam.layout(seam.load().seam_node_layout)
    assert len(mine) == 22 and mine == theirs


def test_hip_table_covers_the_path():
    if not seam.have():
        pytest.skip("oracle/_ref/libseam_ref.so not built (reference tree absent)")
    lib = seam.load()
    absent = {4, 5, 6, 18, 20, 31}    # softmax family: not on the path; 20, 31: nullptr in the reference's tables too
    for code in range(37):
        assert lib.seam_hip_has(code) == (0 if code in absent else 1), code
        if code not in (20, 31):
            assert lib.seam_cpu_has(code) == 1, code
    assert lib.seam_hip_has(37) == 0 and lib.seam_hip_has(511) == 0

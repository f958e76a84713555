"""Compile the HIP sources under csrc/ for gfx950 into lib/libdcgan_hip.so (and the C++ host
mirror under host/ into lib/libdcgan_host.so when present).

    python dcgan-cuda_amd/build.py          # or: from build import build; build()

hipcc cross-compiles without a GPU.  The objects are rebuilt every time build() is called.
"""
import concurrent.futures
import glob
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
HOST = os.path.join(HERE, "host")
LIBDIR = os.path.join(HERE, "lib")
OBJDIR = os.path.join(HERE, "build")
LIB = os.path.join(LIBDIR, "libdcgan_hip.so")
HOSTLIB = os.path.join(LIBDIR, "libdcgan_host.so")

HIPCC = os.environ.get("HIPCC", shutil.which("hipcc") or "/opt/rocm/bin/hipcc")
# packed fp32 VALU ops are switched off for device code (they have miscomputed on these machines)
HIPFLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
            "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
            "-I" + os.path.join(ROOT, "include"), "-I" + CSRC]


def _run(cmd):
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("command failed: %s\n%s\n%s" % (" ".join(cmd), res.stdout, res.stderr))
    return res.stderr


def build(verbose=False, jobs=8):
    os.makedirs(LIBDIR, exist_ok=True)
    os.makedirs(OBJDIR, exist_ok=True)
    srcs = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    objs = [os.path.join(OBJDIR, os.path.basename(s)[:-4] + ".o") for s in srcs]
    cmds = [[HIPCC] + HIPFLAGS + ["-c", s, "-o", o] for s, o in zip(srcs, objs)]
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        for warn in ex.map(_run, cmds):
            if verbose and warn.strip():
                print(warn, file=sys.stderr)
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs)
    host_srcs = sorted(glob.glob(os.path.join(HOST, "*.cc")))
    if host_srcs:
        _run(["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wextra", "-pthread",
              "-I" + os.path.join(ROOT, "include"), "-I" + HOST, "-o", HOSTLIB] + host_srcs +
             ["-L" + LIBDIR, "-ldcgan_hip", "-Wl,-rpath,$ORIGIN"])
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))

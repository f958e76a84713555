"""Weights I/O (numpy .npz and the plain binary format), training-state persistence and the image
helpers of the host library, without a GPU (RT_MODE=CPU in a child process, the oracle as backend).
The checks themselves are in io_roundtrip.py."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_weights_state_and_images_round_trip(tmp_path):
    import __graft_entry__ as ge
    pkg = ge.load_package()
    if not (os.path.exists(pkg.hostabi.LIB_PATH) and os.path.exists(os.path.join(ROOT, "oracle", "liboracle_backend.so"))):
        ge.build()
    env = dict(os.environ, RT_MODE="CPU", OMP_NUM_THREADS="8")
    res = subprocess.run([sys.executable, os.path.join(ROOT, "tests", "io_roundtrip.py"), str(tmp_path)],
                         env=env, timeout=900, capture_output=True, text=True)
    assert res.returncode == 0, res.stdout[-2000:] + res.stderr[-4000:]
    assert "io round trips ok" in res.stdout

"""The C-ABI library loads without a GPU and exports every symbol include/dcgan_hip.h declares
(no compute call is made here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__ as ge
    p = ge.load_package()
    if not os.path.exists(p.hipabi.LIB_PATH):
        ge.build()
    return p


def declared():
    hdr = open(os.path.join(ROOT, "include", "dcgan_hip.h")).read()
    hdr = re.sub(r"/\*.*?\*/", "", hdr, flags=re.S)
    return sorted(set(re.findall(r"\b(dh_\w+)\s*\(", hdr)))


def test_every_declared_symbol_is_exported(pkg):
    lib = ctypes.CDLL(pkg.hipabi.LIB_PATH)
    names = declared()
    assert len(names) >= 45
    for n in names:
        assert hasattr(lib, n), n


def test_binding_covers_header(pkg):
    assert pkg.hipabi.exported_symbols() == declared()
    lib = pkg.load()
    assert b"gfx950" in lib.dh_version()


def test_missing_library_is_loud(pkg, monkeypatch):
    monkeypatch.setattr(pkg.hipabi, "_lib", None)
    monkeypatch.setattr(pkg.hipabi, "LIB_PATH", "/nonexistent/libdcgan_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        pkg.hipabi.load()


def test_fastdiv_host_model():
    """The magic-number division the kernels use for index decoding, modelled in Python
    (same constants as dh::FastDiv), against exact division."""
    import random
    random.seed(1)

    def consts(d):
        l = 0
        while (1 << l) < d:
            l += 1
        return ((1 << 32) * ((1 << l) - d)) // d + 1, l

    for d in [1, 2, 3, 5, 7, 25, 64, 75, 100, 127, 128, 1600, 6400, 65536, 262144, 2 ** 31 - 1] + \
            [random.randrange(1, 2 ** 31) for _ in range(200)]:
        mul, sh = consts(d)
        assert mul < 2 ** 32
        for n in [0, 1, d - 1, d, d + 1, 2 * d - 1, 2 ** 31 - 1] + [random.randrange(0, 2 ** 31) for _ in range(50)]:
            if n < 0 or n >= 2 ** 31:
                continue
            q = ((((n * mul) >> 32) + n) & 0xFFFFFFFF) >> sh
            assert q == n // d, (n, d)

"""The .npz reader behind load_vars / load_state on damaged and hostile archives: every one must end
in the reader's own error, never in an out-of-bounds read or a huge allocation.  No GPU, no model: the
reader is reached through dg_npz_inspect."""
import os
import struct

import numpy as np
import pytest


@pytest.fixture(scope="module")
def H():
    import __graft_entry__ as ge
    pkg = ge.load_package()
    if not os.path.exists(pkg.hostabi.LIB_PATH):
        ge.build()
    return pkg.hostabi


@pytest.fixture()
def good(tmp_path):
    path = str(tmp_path / "good.npz")
    np.savez(path, arr_0=np.arange(12, dtype=np.float32).reshape(3, 4), arr_1=np.ones(5, np.float64))
    return path


def patched(path, out, edit):
    raw = bytearray(open(path, "rb").read())
    edit(raw)
    open(out, "wb").write(bytes(raw))
    return out


def test_a_sound_archive_is_read(H, good):
    assert H.npz_inspect(good) == (2, 17)


@pytest.mark.parametrize("keep", [0, 10, 21, 60, 150, -30, -5])
def test_truncated_archives_are_refused(H, good, tmp_path, keep):
    raw = open(good, "rb").read()
    cut = str(tmp_path / "cut.npz")
    open(cut, "wb").write(raw[:keep] if keep >= 0 else raw[:len(raw) + keep])
    with pytest.raises(H.HostError, match="npz:"):
        H.npz_inspect(cut)


def test_header_without_a_shape_tuple(H, good, tmp_path):
    def edit(raw):
        i = raw.index(b"'shape': (")
        raw[i + 9:i + 10] = b"["          # no '(' any more
        j = raw.index(b")", i)
        raw[j:j + 1] = b"]"
    with pytest.raises(H.HostError, match="shape"):
        H.npz_inspect(patched(good, str(tmp_path / "noshape.npz"), edit))


def test_header_without_quotes_around_the_dtype(H, good, tmp_path):
    def edit(raw):
        i = raw.index(b"'<f4'")
        raw[i:i + 5] = b" <f4 "
    with pytest.raises(H.HostError, match="descr|dtype"):
        H.npz_inspect(patched(good, str(tmp_path / "nodescr.npz"), edit))


def test_oversized_shape(H, good, tmp_path):
    """A shape whose element count times 4 wraps around 2^64 to the payload's size must not pass."""
    def edit(raw):
        i = raw.index(b"'shape': (3, 4)")
        # header text is padded with blanks: room for a longer tuple of the same total length
        end = raw.index(b"\n", i)
        text = b"'shape': (4611686018427387907, 4), }"
        raw[i:end] = text + b" " * (end - i - len(text))
    with pytest.raises(H.HostError, match="does not match its shape"):
        H.npz_inspect(patched(good, str(tmp_path / "wrap.npz"), edit))


def test_member_name_running_past_the_directory(H, good, tmp_path):
    def edit(raw):
        i = raw.index(b"PK\x01\x02")
        raw[i + 28:i + 30] = struct.pack("<H", 0xFFF0)    # name length far beyond the directory
    with pytest.raises(H.HostError, match="central directory"):
        H.npz_inspect(patched(good, str(tmp_path / "name.npz"), edit))


def test_member_size_beyond_the_file(H, good, tmp_path):
    def edit(raw):
        i = raw.index(b"PK\x01\x02")
        raw[i + 20:i + 24] = struct.pack("<I", 0xF0000000)   # compressed and original size: 3.75 GiB
        raw[i + 24:i + 28] = struct.pack("<I", 0xF0000000)
    with pytest.raises(H.HostError, match="truncated member"):
        H.npz_inspect(patched(good, str(tmp_path / "size.npz"), edit))


def test_directory_offset_beyond_the_file(H, good, tmp_path):
    def edit(raw):
        i = raw.rindex(b"PK\x05\x06")
        raw[i + 16:i + 20] = struct.pack("<I", 0x7FFFFFFF)
    with pytest.raises(H.HostError, match="outside the file"):
        H.npz_inspect(patched(good, str(tmp_path / "cdoff.npz"), edit))


def test_compressed_archives_are_refused_with_advice(H, tmp_path):
    path = str(tmp_path / "z.npz")
    np.savez_compressed(path, arr_0=np.zeros(100, np.float32))
    with pytest.raises(H.HostError, match="savez"):
        H.npz_inspect(path)

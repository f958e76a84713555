"""Child-process script of test_host_io.py: weight files, training state and image helpers of the
host library, in RT_MODE=CPU with the oracle as backend (the program mode is process-wide).

    python tests/io_roundtrip.py <scratch directory>

Exits non-zero (assertion) on the first mismatch.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import __graft_entry__ as ge  # noqa: E402
import dcgan_reference as dr  # noqa: E402


def read_ppm(path):
    raw = open(path, "rb").read()
    magic, w, h, maxval = raw.split(None, 4)[:4]
    assert magic == b"P6" and maxval == b"255"
    w, h = int(w), int(h)
    return np.frombuffer(raw[len(raw) - w * h * 3:], np.uint8).reshape(h, w, 3)


def main(tmp):
    pkg = ge.load_package()
    H = pkg.hostabi
    model = H.DcganModel(1, 3, "CPU", os.path.join(ROOT, "oracle", "liboracle_backend.so"))
    names = H.VAR_NAMES
    shapes = H.var_shapes()
    w, z, x = dr.synthetic(1, 11, shapes)
    for n in names:
        model.set_var(n, w[n])

    # ---- trainable variables <-> numpy .npz -------------------------------------------------
    p1 = os.path.join(tmp, "weights.npz")
    model.save_vars(p1)
    with np.load(p1) as f:
        assert sorted(f.files, key=lambda s: int(s[4:])) == ["arr_%d" % i for i in range(len(names))]
        saved = [f["arr_%d" % i] for i in range(len(names))]
    by_size = sorted(int(np.prod(shapes[n])) for n in names)
    assert sorted(a.size for a in saved) == by_size
    for a in saved:
        assert a.dtype == np.float32
        # creation order differs from VAR_NAMES order: match by content
        assert any(a.shape == tuple(shapes[n]) and np.array_equal(a, w[n]) for n in names), a.shape
    # numpy writes, the library reads: float32, float64 (converted), any member order
    new = [(a * 2 + 1).astype(np.float32) for a in saved]
    p2 = os.path.join(tmp, "from_numpy.npz")
    np.savez(p2, **{"arr_%d" % i: (a.astype(np.float64) if i % 2 else a) for i, a in reversed(list(enumerate(new)))})
    model.load_vars(p2)
    p3 = os.path.join(tmp, "again.npz")
    model.save_vars(p3)
    with np.load(p3) as f:
        for i, a in enumerate(new):
            np.testing.assert_array_equal(f["arr_%d" % i], a)
    # compressed archives are refused with a message that says why
    p4 = os.path.join(tmp, "compressed.npz")
    np.savez_compressed(p4, *new)
    try:
        model.load_vars(p4)
        raise AssertionError("a compressed archive was accepted")
    except H.HostError as e:
        assert "compressed" in str(e), str(e)
    try:
        np.savez(os.path.join(tmp, "short.npz"), *new[:-1])
        model.load_vars(os.path.join(tmp, "short.npz"))
        raise AssertionError("an archive with too few arrays was accepted")
    except H.HostError as e:
        assert "arrays" in str(e), str(e)
    # the plain binary format still round-trips
    p5 = os.path.join(tmp, "weights.bin")
    model.save_vars(p5)
    for n in names:
        model.set_var(n, np.zeros(shapes[n], np.float32))
    model.load_vars(p5)
    model.save_vars(p3)
    with np.load(p3) as f:
        for i, a in enumerate(new):
            np.testing.assert_array_equal(f["arr_%d" % i], a)

    # ---- training state: a reloaded run continues exactly as the original -----------------
    for n in names:
        model.set_var(n, w[n])
    model.set_inputs(z, x)
    model.d_step()
    ps = os.path.join(tmp, "state.npz")
    model.save_state(ps)
    with np.load(ps) as f:
        t = f["adam_t"]
        n_vars = len([k for k in f.files if k.startswith("var_")])
    assert n_vars == 3 * len(names), n_vars            # every variable plus two moment estimates each
    assert t.shape == (len(names),) and sorted(t.tolist()) == [0.0] * 10 + [1.0] * 10, t
    model.d_step()
    model.g_step()
    after = {n: model.var(n) for n in names}
    model.load_state(ps)
    with np.load(ps) as f:
        pass
    model.d_step()
    model.g_step()
    for n in names:
        np.testing.assert_array_equal(model.var(n), after[n], err_msg=n)

    # ---- images --------------------------------------------------------------------------------
    rng = np.random.default_rng(5)
    pix = rng.integers(0, 256, (4, 64, 64, 3), dtype=np.uint8)
    pix[0, 0, 0] = (0, 255, 128)
    norm = H.images_normalize(pix)
    np.testing.assert_array_equal(norm, (pix.astype(np.float64) / 127.5 - 1.0).astype(np.float32))
    assert norm.min() == -1.0 and norm.max() == 1.0
    pm = os.path.join(tmp, "mosaic.ppm")
    H.images_save_samples(norm, 2, 2, pm)
    mosaic = read_ppm(pm)
    assert mosaic.shape == (128, 128, 3)
    expect = ((norm.astype(np.float64) + 1.0) * 127.5).astype(np.uint8)   # truncation, as the reference
    for j in range(2):
        for i in range(2):
            np.testing.assert_array_equal(mosaic[j * 64:(j + 1) * 64, i * 64:(i + 1) * 64], expect[j * 2 + i])
    assert np.abs(mosaic[:64, :64].astype(int) - pix[0].astype(int)).max() <= 1
    # out-of-range values are clamped
    H.images_save_samples(np.full((1, 64, 64, 3), 3.0, np.float32), 1, 1, pm)
    assert read_ppm(pm).min() == 255
    H.images_save_samples(np.full((1, 64, 64, 3), -3.0, np.float32), 1, 1, pm)
    assert read_ppm(pm).max() == 0
    # a directory of <index>.ppm files -> normalised batch
    d = os.path.join(tmp, "celeba_norm")
    os.makedirs(d, exist_ok=True)
    for k in range(3):
        with open(os.path.join(d, "%06d.ppm" % (k + 7)), "wb") as f:
            f.write(b"P6\n# a comment line\n64 64\n255\n" + pix[k].tobytes())
    batch = H.images_load(d, 7, 10)
    np.testing.assert_array_equal(batch, norm[:3])
    try:
        H.images_load(d, 0, 1)
        raise AssertionError("a missing image was accepted")
    except H.HostError as e:
        assert "cannot open" in str(e), str(e)
    model.close()
    print("io round trips ok")


if __name__ == "__main__":
    main(sys.argv[1])

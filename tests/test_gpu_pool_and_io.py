"""The parts of the host library around the hot path, on the GPU: the pooled tensor allocator behind
tensor_alloc / tensor_free (the reference calls cudaMalloc per operator output at every Op::compile,
src/ops/conv2d.cu:49-79, src/ops/graph.cu:104-120), the scratch-arena reservation, weights and training
state written from and read back into device memory (src/ops/graph.cu:326-361), and the image feed
(src/datasets/celeba.cu:16-68) into a discriminator step."""
import os

import numpy as np
import pytest

import dcgan_reference as dr

pytestmark = pytest.mark.gpu
SEED = 7


@pytest.fixture(scope="module")
def pkg():
    import __graft_entry__ as ge
    return ge.load_package()


def make_model(pkg, batch, fusion=True):
    model = pkg.hostabi.DcganModel(batch, SEED, "GPU")
    model.set_fusion(fusion)
    w, z, x = dr.synthetic(batch, SEED, pkg.hostabi.var_shapes())
    for name, val in w.items():
        model.set_var(name, val)
    model.set_inputs(z, x)
    return model


def test_pool_blocks_are_aligned_reused_and_merged(pkg):
    A = pkg.hipabi
    lib = A.load()
    import ctypes as C

    def alloc(n):
        p = C.c_void_p()
        A.check(lib.dh_pool_alloc(C.byref(p), n))
        assert p.value % 256 == 0
        return p.value

    A.check(lib.dh_pool_reserve(8 << 20))
    before = A.pool_stats()
    a, b, c = alloc(1 << 20), alloc(3 << 20), alloc(1000)
    assert len({a, b, c}) == 3
    data = np.arange(1 << 18, dtype=np.float32)
    A.check(lib.dh_memcpy_h2d(a, data.ctypes.data, data.nbytes))
    A.check(lib.dh_memcpy_h2d(b, data.ctypes.data, data.nbytes))
    back = np.empty_like(data)
    A.check(lib.dh_memcpy_d2h(back.ctypes.data, a, data.nbytes))
    np.testing.assert_array_equal(back, data)
    mid = A.pool_stats()
    assert mid["in_use"] - before["in_use"] == (1 << 20) + (3 << 20) + 1024
    # b then a come back: the two ranges merge, and a block as large as both fits where they were
    A.check(lib.dh_pool_free(b))
    A.check(lib.dh_pool_free(a))
    d = alloc(4 << 20)
    assert d == min(a, b)
    A.check(lib.dh_pool_free(d))
    A.check(lib.dh_pool_free(c))
    after = A.pool_stats()
    assert after["hipmallocs"] == before["hipmallocs"] and after["in_use"] == before["in_use"]
    with pytest.raises(A.HipError, match="not a live block"):
        A.check(lib.dh_pool_free(c))


def test_a_reservation_is_one_range_not_a_sum_of_fragments(pkg):
    """Idle fragments that add up to the reserved size do not count: after dh_pool_reserve(n) a block of n
    bytes is served without a hipMalloc."""
    A = pkg.hipabi
    lib = A.load()
    import ctypes as C

    def alloc(n):
        p = C.c_void_p()
        A.check(lib.dh_pool_alloc(C.byref(p), n))
        return p.value

    mib = 1 << 20
    blocks = [alloc(2 * mib) for _ in range(8)]
    for b in blocks[::2]:              # every other block back: 8 MiB idle in pieces of 2 MiB (plus what was idle before)
        A.check(lib.dh_pool_free(b))
    big = 700 * mib                    # larger than any range a batch-64 model leaves idle
    A.check(lib.dh_pool_reserve(big))
    before = A.pool_stats()
    assert before["held"] - before["in_use"] >= big
    p = alloc(big)
    assert A.pool_stats()["hipmallocs"] == before["hipmallocs"]
    for b in blocks[1::2] + [p]:
        A.check(lib.dh_pool_free(b))
    A.check(lib.dh_pool_trim())


def test_training_loop_and_a_rebuild_at_another_batch_allocate_nothing(pkg):
    """After the first iteration neither the tensor pool nor the scratch arenas grow; a model torn down
    and built again at a smaller batch (every operator lowered anew, at other shapes) is served from the
    memory already held."""
    A = pkg.hipabi
    lib = A.load()
    model = make_model(pkg, 64)
    try:
        model.d_step(), model.g_step()
        pool, arena = A.pool_stats(), lib.dh_workspace_bytes()
        assert pool["hipmallocs"] >= 1 and pool["in_use"] > 100 << 20
        for _ in range(3):
            model.d_step(want_loss=False), model.g_step(want_loss=False)
        model.sync()
        assert A.pool_stats()["hipmallocs"] == pool["hipmallocs"]
        assert lib.dh_workspace_bytes() == arena
    finally:
        model.set_fusion(False)
        model.close()
    idle = A.pool_stats()
    assert idle["held"] == pool["held"] and idle["in_use"] < pool["in_use"]
    model = make_model(pkg, 32)
    try:
        loss = model.d_step()
        model.g_step()
        assert np.isfinite(loss)
        assert A.pool_stats()["hipmallocs"] == pool["hipmallocs"]
    finally:
        model.set_fusion(False)
        model.close()


def test_workspace_reservation_keeps_the_arena_from_growing(pkg):
    A = pkg.hipabi
    lib = A.load()
    A.check(lib.dh_workspace_reserve(160 << 20))
    held = lib.dh_workspace_bytes()
    assert held >= 160 << 20
    be = pkg.HipBackend(0)
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (64, 8, 8, 256)).astype(np.float32)
    dy = rng.uniform(-1, 1, (64, 4, 4, 512)).astype(np.float32)
    be.conv2d_kernel_grad(dy, x, 2, (3, 3))          # a split launch: its slices live in the arena
    assert lib.dh_workspace_bytes() == held


def snapshot(model, H):
    return {n: model.var(n).copy() for n in H.VAR_NAMES}


def test_training_state_round_trip_on_the_device(pkg, tmp_path):
    """Two fused iterations without reading a loss back (the runs are still queued when save_state reads
    the tensors), the state saved, two more iterations; then the state loaded back into device memory and
    the same two iterations again: identical to the bit, parameters and losses, which also pins the Adam
    moments and step counters that the file carries.  The weights-only file round-trips likewise."""
    H = pkg.hostabi
    model = make_model(pkg, 16)
    try:
        for _ in range(2):
            model.d_step(want_loss=False), model.g_step(want_loss=False)
        state, weights = str(tmp_path / "state.npz"), str(tmp_path / "weights.npz")
        model.save_state(state)
        model.save_vars(weights)
        at_save = snapshot(model, H)
        first = [(model.d_step(), model.g_step()) for _ in range(2)]
        after_first = snapshot(model, H)
        assert any(not np.array_equal(at_save[n], after_first[n]) for n in H.VAR_NAMES)
        model.load_state(state)
        for n, v in snapshot(model, H).items():
            np.testing.assert_array_equal(v, at_save[n], err_msg=n)
        second = [(model.d_step(), model.g_step()) for _ in range(2)]
        assert first == second
        for n, v in snapshot(model, H).items():
            np.testing.assert_array_equal(v, after_first[n], err_msg=n)
        model.load_vars(weights)
        for n, v in snapshot(model, H).items():
            np.testing.assert_array_equal(v, at_save[n], err_msg=n)
        with np.load(weights) as f:
            assert len(f.files) == len(H.VAR_NAMES)
    finally:
        model.set_fusion(False)
        model.close()


def test_images_from_files_into_a_discriminator_step(pkg, tmp_path, orc):
    """8-bit images written as <index>.ppm, loaded and normalised by the library (pix / 127.5 - 1), fed to
    the device and run through a discriminator step: the first layer's output equals the oracle's on the
    same normalised batch, and the mosaic of generated samples is written back as a PPM."""
    H, A = pkg.hostabi, pkg.hipabi
    rng = np.random.default_rng(21)
    batch = 8
    pix = rng.integers(0, 256, (batch, 64, 64, 3), dtype=np.uint8)
    for i in range(batch):
        with open(tmp_path / ("%06d.ppm" % (i + 1)), "wb") as f:
            f.write(b"P6\n64 64\n255\n" + pix[i].tobytes())
    x = H.images_load(str(tmp_path), 1, batch + 1)
    np.testing.assert_array_equal(x, (pix.astype(np.float64) / 127.5 - 1.0).astype(np.float32))   # formed in double, as the reference does
    model = make_model(pkg, batch)
    try:
        w, z, _ = dr.synthetic(batch, SEED, H.var_shapes())
        model.set_inputs(z, x)
        got = model.eval("d_real_l0").reshape(batch, 32, 32, 64)
        exp = orc.relu_leaky(orc.bias_add(orc.conv2d(x, w["d0_w"], (2, 2)), w["d0_b"]), 0.2)
        np.testing.assert_allclose(got, exp, rtol=1e-4, atol=1e-5)
        assert np.isfinite(model.d_step())
        img = model.generate()
        out = str(tmp_path / "samples.ppm")
        H.images_save_samples(img, 4, 2, out)
        raw = open(out, "rb").read()
        assert raw.startswith(b"P6") and len(raw) > 4 * 2 * 64 * 64 * 3
    finally:
        model.set_fusion(False)
        model.close()


def test_inputs_handed_to_the_run_equal_resident_inputs(pkg):
    """The reference's loop passes z and the image batch to every run (dcgan/main.cu:378-391); here such
    inputs are staged and copied inside the run, in front of the first step that reads them.  Three
    iterations fed that way -- with fresh inputs each time, losses read and not read -- against the same
    iterations on inputs made resident beforehand: identical losses and parameters."""
    H = pkg.hostabi
    rng = np.random.default_rng(5)
    batch = 16
    zs = [rng.uniform(-1, 1, (batch, 100)).astype(np.float32) for _ in range(3)]
    xs = [rng.uniform(-1, 1, (batch, 64, 64, 3)).astype(np.float32) for _ in range(3)]
    results = []
    for fed in (False, True):
        model = make_model(pkg, batch)
        try:
            losses = []
            for i, (z, x) in enumerate(zip(zs, xs)):
                want = i != 1
                if fed:
                    zc, xc = z.copy(), x.copy()
                    losses.append((model.d_step(want, z=zc, x=xc), model.g_step(want, z=zc)))
                    zc[:], xc[:] = 7.0, 7.0      # the buffers are the caller's again once the call has returned
                else:
                    model.set_inputs(z, x)
                    losses.append((model.d_step(want), model.g_step(want)))
            results.append((losses, snapshot(model, H)))
        finally:
            model.set_fusion(False)
            model.close()
    assert results[0][0] == results[1][0]
    assert all(np.isfinite(v) for pair in results[0][0] for v in pair if v is not None)
    for n in H.VAR_NAMES:
        np.testing.assert_array_equal(results[0][1][n], results[1][1][n], err_msg=n)

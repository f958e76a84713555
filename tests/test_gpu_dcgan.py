"""Whole-network parity, layer by layer, in the manner of the reference's test_dcgan_generator /
test_dcgan_discriminator (which export every layer, the loss and all dW/db): the DCGAN evaluated
through the operator graph on the HIP backend against the same graph on the CPU oracle backend,
on identical seeded weights and inputs -- unfused and with the fused launches."""
import os
import subprocess
import sys

import numpy as np
import pytest

import dcgan_reference as dr
from common import RTOL, ATOL

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BATCH, SEED = 2, 7


@pytest.fixture(scope="module")
def cpu_dump(tmp_path_factory):
    path = str(tmp_path_factory.mktemp("dcgan") / "cpu.npz")
    env = dict(os.environ, RT_MODE="CPU", OMP_NUM_THREADS="16")
    subprocess.run([sys.executable, os.path.join(ROOT, "tests", "dcgan_reference.py"), str(BATCH), str(SEED), path],
                   check=True, env=env, timeout=600)
    return dict(np.load(path))


def gpu_dump(fusion):
    """fusion: False (one launch per instruction), True (fused launches, the two discriminator towers'
    convolutions paired), "unpaired" (fused launches, every convolution on its own)."""
    import __graft_entry__ as ge
    pkg = ge.load_package()
    model = pkg.hostabi.DcganModel(BATCH, SEED, "GPU")
    try:
        model.set_fusion(bool(fusion))
        model.set_pairing(fusion != "unpaired")
        w, z, x = dr.synthetic(BATCH, SEED, pkg.hostabi.var_shapes())
        for name, val in w.items():
            model.set_var(name, val)
        model.set_inputs(z, x)
        return dr.collect(model), model.last_schedule_size()
    finally:
        model.set_fusion(False)
        model.set_pairing(True)
        model.close()


def test_paired_plan_is_shorter():
    """With pairing the discriminator step issues ten launches fewer: layers 1-3 forward, input
    gradient and filter gradient of the two towers each become one launch, and so does the image
    layer's filter gradient."""
    import __graft_entry__ as ge
    pkg = ge.load_package()
    counts = {}
    for pairing in (True, False):
        model = pkg.hostabi.DcganModel(BATCH, SEED, "GPU")
        try:
            model.set_fusion(True)
            model.set_pairing(pairing)
            w, z, x = dr.synthetic(BATCH, SEED, pkg.hostabi.var_shapes())
            for name, val in w.items():
                model.set_var(name, val)
            model.set_inputs(z, x)
            model.d_step()
            counts[pairing] = model.last_launch_count()
        finally:
            model.set_fusion(False)
            model.set_pairing(True)
            model.close()
    assert counts[False] - counts[True] == 10, counts


@pytest.mark.parametrize("fusion", [False, True, "unpaired"])
def test_dcgan_layers_losses_gradients_and_one_adam_iteration(cpu_dump, fusion):
    print("fusion", fusion, flush=True)
    got, _ = gpu_dump(fusion)
    assert set(got) == set(cpu_dump)
    for key in sorted(cpu_dump):
        exp = cpu_dump[key].reshape(-1)
        g = got[key].reshape(-1)
        if key.startswith("after_"):
            # parameters after one Adam step: the step is lr*m/(sqrt(v)+eps) ~ lr*sign(g); where a
            # gradient is ~0 its sign is noise, so compare with the step size as absolute tolerance
            np.testing.assert_allclose(g, exp, rtol=RTOL, atol=4.1e-4, err_msg=key)
            assert np.mean(np.abs(g - exp) > 1e-5) < 0.02, key
        else:
            scale = max(1.0, float(np.abs(exp).max()))
            np.testing.assert_allclose(g, exp, rtol=RTOL, atol=ATOL * scale, err_msg=key)


def test_generate_and_argmax_bit_exact(cpu_dump):
    """The generated images agree to tolerance and their per-pixel argmax over channels is identical."""
    import __graft_entry__ as ge
    pkg = ge.load_package()
    model = pkg.hostabi.DcganModel(BATCH, SEED, "GPU")
    try:
        w, z, x = dr.synthetic(BATCH, SEED, pkg.hostabi.var_shapes())
        for name, val in w.items():
            model.set_var(name, val)
        model.set_inputs(z, x)
        img = model.generate()
    finally:
        model.close()
    exp = cpu_dump["g_out"].reshape(img.shape)
    np.testing.assert_allclose(img, exp, rtol=RTOL, atol=ATOL)
    margin = np.sort(exp, axis=-1)
    clear = (margin[..., -1] - margin[..., -2]) > 1e-5   # exclude numerical ties
    assert np.array_equal(img.argmax(-1)[clear], exp.argmax(-1)[clear])
    assert clear.mean() > 0.95


def test_generator_at_batch_4096_is_batch_invariant(cpu_dump):
    """Generator-only inference at batch 4096 (largest activation [4096,32,32,64], 1.07 GB): too
    large for the oracle, so the check is a property -- an image does not depend on the batch it
    is generated in.  The first BATCH latent vectors are the oracle-checked ones; their images
    must agree with the oracle's to tolerance, and images of repeated latent vectors elsewhere in
    the batch (its last rows, the rows across the 2 GiB byte offset of the largest activation)
    must agree with the images of the rows they repeat."""
    import __graft_entry__ as ge
    pkg = ge.load_package()
    big = 4096
    w, z, _ = dr.synthetic(BATCH, SEED, pkg.hostabi.var_shapes())
    rng = np.random.default_rng(5)
    zb = rng.uniform(-1, 1, (big, 100)).astype(np.float32)
    zb[:BATCH] = z
    copies = {big - 1: 17, big - 2: 1000, 2048: 3, 2047: 4000}     # row -> row whose z it repeats
    for dst, src in copies.items():
        zb[dst] = zb[src]
    model = pkg.hostabi.DcganModel(big, SEED, "GPU")
    try:
        model.set_fusion(True)
        for name, val in w.items():
            model.set_var(name, val)
        model.set_inputs(z=zb)
        model.generate(to_host=False)          # device-resident pass, as the benchmark runs it
        img = model.generate()
    finally:
        model.set_fusion(False)
        model.close()
    assert np.isfinite(img).all()
    exp = cpu_dump["g_out"].reshape(BATCH, 64, 64, 3)
    np.testing.assert_allclose(img[:BATCH], exp, rtol=RTOL, atol=ATOL)
    for dst, src in copies.items():
        np.testing.assert_allclose(img[dst], img[src], rtol=RTOL, atol=ATOL)
    assert len({img[i].tobytes() for i in range(0, big, 97)}) == len(range(0, big, 97))   # rows differ

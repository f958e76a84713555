"""The host library (operator graph, differentiation, rt::Node packing, scheduling) exercised
without a GPU: RT_MODE=CPU with the oracle plugged in as backend, in a child process because the
program mode is process-wide.  The whole DCGAN -- every layer output, both losses and the gradient
of every parameter -- is pinned against an independent float64 torch restatement."""
import os
import subprocess
import sys

import numpy as np
import pytest

import dcgan_reference as dr

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def cpu_dump(tmp_path_factory):
    import __graft_entry__ as ge
    pkg = ge.load_package()
    if not (os.path.exists(pkg.hostabi.LIB_PATH) and os.path.exists(os.path.join(ROOT, "oracle", "liboracle_backend.so"))):
        ge.build()
    path = str(tmp_path_factory.mktemp("dcgan") / "cpu.npz")
    env = dict(os.environ, RT_MODE="CPU", OMP_NUM_THREADS="8")
    subprocess.run([sys.executable, os.path.join(ROOT, "tests", "dcgan_reference.py"), "2", "7", path],
                   check=True, env=env, timeout=600)
    return dict(np.load(path))


def test_dcgan_forward_losses_and_all_gradients_vs_torch_f64(cpu_dump):
    import __graft_entry__ as ge
    shapes = ge.load_package().hostabi.var_shapes()
    w, z, x = dr.synthetic(2, 7, shapes)
    ref = dr.torch_dcgan(w, z, x)
    assert len(ref) >= 40
    for key, exp in ref.items():
        got = cpu_dump[key].reshape(-1).astype(np.float64)
        tol = 2e-5 * max(1.0, float(np.abs(exp).max()))
        np.testing.assert_allclose(got, exp, rtol=2e-4, atol=tol, err_msg=key)


def test_labelled_discriminator_pass_vs_torch_f64(tmp_path):
    """The discriminator alone on labelled images (random 0/1 labels): layers, logits, loss, all dW / db and
    the gradient of the input images."""
    import __graft_entry__ as ge
    path = str(tmp_path / "disc.npz")
    env = dict(os.environ, RT_MODE="CPU", OMP_NUM_THREADS="8")
    subprocess.run([sys.executable, os.path.join(ROOT, "tests", "dcgan_reference.py"), "3", "11", path, "disc"],
                   check=True, env=env, timeout=600)
    got = dict(np.load(path))
    w, _, x = dr.synthetic(3, 11, ge.load_package().hostabi.var_shapes())
    y = dr.labels(3, 11)
    ref = dr.torch_disc(w, x, y)
    assert set(ref) == set(got) and len(ref) == 17
    for key, exp in ref.items():
        tol = 2e-5 * max(1.0, float(np.abs(exp).max()))
        np.testing.assert_allclose(got[key].reshape(-1).astype(np.float64), exp, rtol=2e-4, atol=tol, err_msg=key)
    assert np.abs(ref["grad_disc_loss_x_real"]).max() > 0


def test_adam_step_moves_parameters_as_the_closed_form_says(cpu_dump):
    """After the first Adam step (m = (1-b1) g, v = (1-b2) g^2, t = 1) every parameter moves by
    lr * sign(g) / (1 + eps / (sqrt(1-b2) |g|)): |delta| ~= 2e-4 wherever |g| >> 3e-7."""
    import __graft_entry__ as ge
    shapes = ge.load_package().hostabi.var_shapes()
    w, _, _ = dr.synthetic(2, 7, shapes)
    for v in dr.D_VARS:
        g = cpu_dump["grad_d_loss_" + v]
        delta = cpu_dump["after_" + v] - w[v].reshape(-1)
        big = np.abs(g) > 1e-4   # eps = 1e-8 then changes the step by < 0.4 %
        assert big.any()
        np.testing.assert_allclose(delta[big], -2e-4 * np.sign(g[big]), rtol=2e-2, atol=2e-6, err_msg=v)


def test_cpu_mode_without_backend_is_an_error(tmp_path):
    """RT_MODE=CPU with nothing registered must throw, not fall back silently."""
    code = ("import sys; sys.path.insert(0, %r); import __graft_entry__ as ge; pkg = ge.load_package();\n"
            "import os; os.environ['RT_MODE']='CPU'\n"
            "lib = pkg.hostabi.load(); h = lib.dg_create(1, 1)\n"
            "print('HANDLE', h, lib.dg_last_error().decode())\n" % ROOT)
    res = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120,
                         env=dict(os.environ, RT_MODE="CPU"))
    assert "HANDLE None" in res.stdout and "only holds the HIP backend" in res.stdout, res.stdout + res.stderr

"""The drop-in seam proved with the reference's own record: every instruction here is made by the
reference's rt::Node::op_* factory (src/runtime/node.cu), executed by this build's
hip::kernels_list[node->type] -- compiled unchanged against the reference's src/runtime/node.hh -- on
device buffers, and compared with the reference's cpu::kernels_list[node->type] on the same host data
(src/gpu/kernels.cu:23-61 and src/gpu/runner.cu:10-18 are what the HIP table replaces).  The two
conv2d_transpose gradients run on VALID-equivalent shapes, the only ones the reference's CPU functions
handle (src/cpu/ops.hxx:808-902)."""
import numpy as np
import pytest

import seam
from common import RTOL, ATOL, same_pad

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def A():
    if not seam.have():
        pytest.fail("oracle/_ref/libseam_ref.so is missing: build() makes it where the reference tree is mounted")
    import __graft_entry__ as ge
    return ge.load_package().hipabi


def rnd(rng, *shape):
    return rng.uniform(-1, 1, shape).astype(np.float32)


def close(got, exp, what, exact=False):
    if exact:
        np.testing.assert_array_equal(got, exp, err_msg=what)
    else:
        scale = max(1.0, float(np.abs(exp).max()))
        np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL * scale, err_msg=what)


CONV_SHAPES = [  # N, H, W, C, kh, kw, O, stride
    (2, 8, 8, 3, 5, 5, 4, 2),
    (3, 9, 7, 6, 3, 3, 5, 2),
    (4, 16, 16, 32, 5, 5, 64, 2),      # buffer-load kernel
    (64, 8, 8, 256, 5, 5, 512, 2),     # discriminator layer 3 at the benchmark's batch
]


@pytest.mark.parametrize("shape", CONV_SHAPES)
def test_conv2d_nodes(A, orc, shape):
    N, H, W, C, kh, kw, O, s = shape
    rng = np.random.default_rng(sum(shape))
    (ph, Ho), (pw, Wo) = same_pad(H, kh, s), same_pad(W, kw, s)
    x, k, dy = rnd(rng, N, H, W, C), rnd(rng, kh, kw, C, O) * 0.1, rnd(rng, N, Ho, Wo, O)
    # At the benchmark's size the reference's CPU loops run ~10 s per forward product and minutes per
    # gradient: there only the forward node goes through the reference's table; the other nodes -- still made
    # by the reference's factories and run through the HIP table -- are compared with the oracle, which the
    # small shapes of this test (and tests/test_oracle_vs_ref.py) tie to the reference's CPU table.
    small = N < 64
    # conv2d: strides, total pads, input dims, filter dims (src/runtime/node.cu:118-141)
    (e, _), (g, _), code = seam.run_both(A, "conv2d", [x, k, None, np.zeros((N, Ho, Wo, O), np.float32), None],
                                         [s, s, ph, pw, N, H, W, C, kh, kw, C, O])
    assert code == 7
    close(g, e, "conv2d")
    if not small:
        pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
        g = seam.run_hip(A, "conv2d_input_grad", [dy, k, None, np.zeros((N, H, W, C), np.float32), None],
                         [s, s, N, Ho, Wo, O, kh, kw, C, O, N, H, W, C])
        close(g, orc.conv2d_input_grad(dy, k, s, (H, W)), "conv2d_input_grad at batch 64")
        g = seam.run_hip(A, "conv2d_kernel_grad", [dy, x, None, np.zeros((kh, kw, C, O), np.float32), None],
                         [s, s, N, Ho, Wo, O, N, H, W, C, ph, pw])
        close(g, orc.conv2d_kernel_grad(dy, x, s, pads, (kh, kw)), "conv2d_kernel_grad at batch 64")
        g = seam.run_hip(A, "conv2d_transpose", [dy, k, None, np.zeros((N, H, W, C), np.float32), None],
                         [N, H, W, C, s, s, N, Ho, Wo, O, kh, kw, C, O])
        close(g, orc.conv2d_transpose(dy, k, (H, W), s), "conv2d_transpose at batch 64")
        # gradients of that transpose (x_t := dy, y_t := x): input gradient = conv2d of dy_t, filter gradient
        # with the roles of the activations exchanged (src/gpu/conv2d.cu:214-307)
        g = seam.run_hip(A, "conv2d_transpose_input_grad", [x, k, None, np.zeros((N, Ho, Wo, O), np.float32), None],
                         [s, s, N, H, W, C, kh, kw, C, O, N, Ho, Wo, O])
        close(g, orc.conv2d_transpose_input_grad(x, k, s, (Ho, Wo)), "conv2d_transpose_input_grad at batch 64")
        g = seam.run_hip(A, "conv2d_transpose_kernel_grad", [x, dy, None, np.zeros((kh, kw, C, O), np.float32), None],
                         [s, s, N, H, W, C, N, Ho, Wo, O, kh, kw, C, O])
        close(g, orc.conv2d_transpose_kernel_grad(x, dy, s, (kh, kw)), "conv2d_transpose_kernel_grad at batch 64")
        return
    # input gradient: strides, dy dims, filter dims, input dims (:171-193)
    (e, _), (g, _), code = seam.run_both(A, "conv2d_input_grad", [dy, k, None, np.zeros((N, H, W, C), np.float32), None],
                                         [s, s, N, Ho, Wo, O, kh, kw, C, O, N, H, W, C])
    assert code == 24
    close(g, e, "conv2d_input_grad")
    # filter gradient: strides, dy dims, input dims, total pads (:195-217)
    (e, _), (g, _), code = seam.run_both(A, "conv2d_kernel_grad", [dy, x, None, np.zeros((kh, kw, C, O), np.float32), None],
                                         [s, s, N, Ho, Wo, O, N, H, W, C, ph, pw])
    assert code == 25
    close(g, e, "conv2d_kernel_grad")
    # conv2d_transpose of dy back onto the input's extent: out dims, strides, input dims, filter dims (:219-243)
    (e, _), (g, _), code = seam.run_both(A, "conv2d_transpose", [dy, k, None, np.zeros((N, H, W, C), np.float32), None],
                                         [N, H, W, C, s, s, N, Ho, Wo, O, kh, kw, C, O])
    assert code == 33
    close(g, e, "conv2d_transpose")


def test_conv2d_transpose_gradient_nodes(A):
    """x_t [2,4,4,3] -> y [2,8,8,2], filter [2,2,2,3], stride 2: no padding either way."""
    rng = np.random.default_rng(5)
    x, k, dy = rnd(rng, 2, 4, 4, 3), rnd(rng, 2, 2, 2, 3), rnd(rng, 2, 8, 8, 2)
    (e, _), (g, _), code = seam.run_both(A, "conv2d_transpose_input_grad", [dy, k, None, np.zeros((2, 4, 4, 3), np.float32), None],
                                         [2, 2, 2, 8, 8, 2, 2, 2, 2, 3, 2, 4, 4, 3])
    assert code == 34
    close(g, e, "conv2d_transpose_input_grad")
    (e, _), (g, _), code = seam.run_both(A, "conv2d_transpose_kernel_grad", [dy, x, None, np.zeros((2, 2, 2, 3), np.float32), None],
                                         [2, 2, 2, 8, 8, 2, 2, 4, 4, 3, 2, 2, 2, 3])
    assert code == 35
    close(g, e, "conv2d_transpose_kernel_grad")


def test_bias_activation_and_loss_nodes(A):
    rng = np.random.default_rng(9)
    rows, cols = 96, 40
    z, d, b = rnd(rng, rows, cols), rnd(rng, rows, cols), rnd(rng, cols)
    n = rows * cols
    out = np.zeros((rows, cols), np.float32)
    cases = [
        ("mat_rvect_add", [z, b, None, out, None], [rows, cols], [], 1, True),
        ("mat_sum_cols", [z, None, None, np.zeros(cols, np.float32), None], [rows, cols], [], 17, False),
        ("mat_sum_rows", [z, None, None, np.zeros(rows, np.float32), None], [rows, cols], [], 16, False),
        ("relu", [z, None, None, out, None], [n], [], 8, True),
        ("relu_leaky", [z, None, None, out, None], [n], [0.2], 9, True),
        ("tanh", [z, None, None, out, None], [n], [], 10, False),
        ("sigmoid", [z, None, None, out, None], [n], [], 2, False),
        ("relu_grad", [z, d, None, out, None], [n], [], 19, True),
        ("leaky_relu_grad", [z, d, None, out, None], [n], [0.2], 30, True),
        ("tanh_grad", [np.tanh(z), d, None, out, None], [n], [], 32, False),
        ("sigmoid_grad", [1 / (1 + np.exp(-z)), d, None, out, None], [n], [], 12, False),
        ("add", [z, d, None, out, None], [n], [], 36, True),
        ("mse", [z, d, None, np.zeros(1, np.float32), None], [rows, cols], [], 3, False),
        ("mse_grad", [z, d, None, out, None], [n], [], 11, False),
        ("sigmoid_cross_entropy", [(z > 0).astype(np.float32), d * 4, None, np.zeros(1, np.float32), None], [n], [], 22, False),
        ("sigmoid_cross_entropy_grad", [(z > 0).astype(np.float32), d * 4, None, out, None], [n], [], 23, False),
    ]
    for op, arrays, ints, floats, want, exact in cases:
        print(op, flush=True)
        (e, _), (g, _), code = seam.run_both(A, op, arrays, ints, floats)
        assert code == want, op
        close(g, e, op, exact)


def test_dense_and_argmax_nodes(A):
    rng = np.random.default_rng(11)
    m, n, p = 64, 100, 48
    a, b, bias = rnd(rng, m, n), rnd(rng, n, p), rnd(rng, p)
    (e, _), (g, _), code = seam.run_both(A, "mat_mat_mul", [a, b, None, np.zeros((m, p), np.float32), None], [m, n, p])
    assert code == 0
    close(g, e, "mat_mat_mul")
    (e, _), (g, _), code = seam.run_both(A, "mat_mul_add", [a, b, bias, np.zeros((m, p), np.float32), None], [m, n, p])
    assert code == 13
    close(g, e, "mat_mul_add")
    # tr(A) B with A stored as [n, m] and B [n, p]: the node carries the extents of the PRODUCT, (m, n, p)
    # (src/cpu/ops.hxx:73-88 reads a[k * m + i])
    at = rnd(rng, n, m)
    (e, _), (g, _), code = seam.run_both(A, "tmat_mat_mul", [at, b, None, np.zeros((m, p), np.float32), None], [m, n, p])
    assert code == 14
    close(g, e, "tmat_mat_mul")
    # A tr(B) with A [m, n], B [p, n]
    bt = rnd(rng, p, n)
    (e, _), (g, _), code = seam.run_both(A, "mat_tmat_mul", [a, bt, None, np.zeros((m, p), np.float32), None], [m, n, p])
    assert code == 15
    close(g, e, "mat_tmat_mul")
    y, y_hat = rnd(rng, 50, 10), rnd(rng, 50, 10)
    y_hat[:20] = y[:20]
    (e, _), (g, _), code = seam.run_both(A, "argmax_acc", [y, y_hat, None, np.zeros(1, np.float32), None], [50, 10])
    assert code == 26
    close(g, e, "argmax_acc", exact=True)
    assert e[0] >= 20


def test_optimiser_nodes(A):
    """In-place instructions: out1 is the variable / moment itself; adam_update's out2 is a HOST pointer
    to the step counter, which the table entry advances on the host (src/gpu/update.cu:81-96)."""
    rng = np.random.default_rng(13)
    n = 5000
    var, g1, m, v = rnd(rng, n), rnd(rng, n), rnd(rng, n) * 0.1, np.abs(rnd(rng, n)) * 0.01
    (e, _), (g, _), code = seam.run_both(A, "moment_update", [g1, None, None, m, None], [n], [0.5, 0.5])
    assert code == 27
    close(g, e, "moment_update", exact=True)
    (e, _), (g, _), code = seam.run_both(A, "moment_update2", [g1, None, None, v, None], [n], [0.999, 0.001])
    assert code == 28
    close(g, e, "moment_update2")
    t = np.array([2.0], np.float32)
    (e, et), (g, gt), code = seam.run_both(A, "adam_update", [m, v, None, var, t], [n], [2e-4, 0.5, 0.999, 1e-8], host_slots=(4,))
    assert code == 29
    assert et[0] == 3.0 and gt[0] == 3.0        # each backend advanced its own copy of the counter once
    close(g, e, "adam_update")
    coeff = np.array([-0.05], np.float32)
    (e, _), (g, _), code = seam.run_both(A, "update", [g1, coeff, None, var, None], [n])
    assert code == 21
    close(g, e, "update")

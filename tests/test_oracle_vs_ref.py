"""The C restatement (oracle/dcgan_oracle.c) against the reference's own CPU operators compiled
into oracle/_ref: BIT-exact on seeded inputs, including the order of the fp32 additions.
Skipped where the reference build is absent (it is produced from /root/reference)."""
import numpy as np
import pytest

from common import rand_conv_inputs, same_pad

SHAPES = [  # N, H, W, C, kh, kw, O, stride
    (2, 8, 8, 3, 5, 5, 4, 2),      # DCGAN-like: 5x5, stride 2, SAME pad (1,2)
    (1, 7, 9, 2, 3, 3, 5, 2),      # odd extents
    (2, 6, 6, 4, 5, 5, 3, 1),      # stride 1, pad (2,2)
    (1, 9, 7, 2, 3, 5, 2, 3),      # stride 3, rectangular filter
    (3, 4, 4, 8, 2, 2, 8, 2),      # pad 0
    (1, 5, 5, 1, 5, 5, 1, 2),
]


def eq(a, b):
    np.testing.assert_array_equal(np.asarray(a), np.asarray(b))


@pytest.mark.parametrize("shape", SHAPES)
def test_conv_ops_bit_exact(orc, ref, shape):
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(7, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    eq(orc.conv2d(x, k, (s, s)), ref.conv2d(x, k, (s, s)))
    eq(orc.conv2d_input_grad(dy, k, s, (H, W)), ref.conv2d_input_grad(dy, k, s, (H, W)))
    eq(orc.conv2d_kernel_grad(dy, x, s, pads), ref.conv2d_kernel_grad(dy, x, s, pads))
    # conv2d_transpose(input := dy, kernel [kh,kw,Cout_t=C,Cin_t=O]) -> [N,H,W,C]
    eq(orc.conv2d_transpose(dy, k, (H, W), s), ref.conv2d_transpose(dy, k, (H, W), s))


def test_transpose_grads_valid_shape_bit_exact(orc, ref):
    """pad_total == 0 (k == stride): the only kind of shape the reference's CPU transpose
    gradients handle; there the identities the oracle follows must equal them."""
    rng = np.random.default_rng(3)
    x = rng.uniform(-1, 1, (2, 4, 4, 3)).astype(np.float32)
    k = rng.standard_normal((2, 2, 2, 3)).astype(np.float32)
    dy = rng.uniform(-1, 1, (2, 8, 8, 2)).astype(np.float32)
    eq(orc.conv2d_transpose_input_grad(dy, k, 2, (4, 4)), ref.conv2d_transpose_input_grad(dy, k, 2, (4, 4)))
    a = orc.conv2d_transpose_kernel_grad(dy, x, 2, (2, 2))
    b = ref.conv2d_transpose_kernel_grad(dy, x, 2, (2, 2))
    np.testing.assert_allclose(a, b, rtol=1e-6, atol=1e-6)  # the reference sums in another order here


def test_elementwise_bit_exact(orc, ref):
    rng = np.random.default_rng(11)
    a = rng.uniform(-3, 3, (37, 19)).astype(np.float32)
    b = rng.uniform(-3, 3, (37, 19)).astype(np.float32)
    a[0, :4] = [0.0, -0.0, 1e-30, -1e-30]
    bias = rng.standard_normal(19).astype(np.float32)
    eq(orc.bias_add(a, bias), ref.bias_add(a, bias))
    eq(orc.bias_grad(a), ref.bias_grad(a))
    eq(orc.mat_sum_rows(a), ref.mat_sum_rows(a))
    for name in ("relu", "tanh", "sigmoid"):
        eq(getattr(orc, name)(a), getattr(ref, name)(a))
    eq(orc.relu_leaky(a, 0.2), ref.relu_leaky(a, 0.2))
    eq(orc.relu_grad(a, b), ref.relu_grad(a, b))
    eq(orc.leaky_relu_grad(a, b, 0.3), ref.leaky_relu_grad(a, b, 0.3))
    t = orc.tanh(a)
    eq(orc.tanh_grad(t, b), ref.tanh_grad(t, b))
    s = orc.sigmoid(a)
    eq(orc.sigmoid_grad(s, b), ref.sigmoid_grad(s, b))
    eq(orc.add(a, b), ref.add(a, b))
    y = (rng.uniform(0, 1, a.shape) > 0.5).astype(np.float32)
    assert orc.sigmoid_cross_entropy(y, a) == ref.sigmoid_cross_entropy(y, a)
    eq(orc.sigmoid_cross_entropy_grad(y, a), ref.sigmoid_cross_entropy_grad(y, a))
    assert orc.mse(a, b) == ref.mse(a, b)
    eq(orc.mse_grad(a, b), ref.mse_grad(a, b))
    assert orc.argmax_acc(a, b) == ref.argmax_acc(a, b)


def test_dense_bit_exact(orc, ref):
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (9, 33)).astype(np.float32)
    w = rng.standard_normal((33, 17)).astype(np.float32)
    b = rng.standard_normal(17).astype(np.float32)
    g = rng.standard_normal((9, 17)).astype(np.float32)
    eq(orc.mat_mul_add(x, w, b), ref.mat_mul_add(x, w, b))
    eq(orc.mm_mul(x, w), ref.mm_mul(x, w))
    eq(orc.tmm_mul(x, g), ref.tmm_mul(x, g))
    eq(orc.mtm_mul(g, w), ref.mtm_mul(g, w))


def test_adam_bit_exact(orc, ref):
    rng = np.random.default_rng(9)
    p = rng.standard_normal(1000).astype(np.float32)
    g = rng.standard_normal(1000).astype(np.float32)
    m = rng.standard_normal(1000).astype(np.float32)
    v = rng.uniform(0, 1, 1000).astype(np.float32)
    eq(orc.moment_update(m, g, 0.5, 0.5), ref.moment_update(m, g, 0.5, 0.5))
    eq(orc.moment_update2(v, g, 0.999, 0.001), ref.moment_update2(v, g, 0.999, 0.001))
    eq(orc.adam_apply(p, m, v, 3e-4, 1e-8), ref.adam_apply(p, m, v, 3e-4, 1e-8))
    eq(orc.vect_update(p, g, -0.1), ref.vect_update(p, g, -0.1))


@pytest.mark.parametrize("mcpu", [False, True])
def test_reference_runtime_runs_the_conv_nodes(ref, mcpu):
    """The node-list path used for the MCPU baseline timing (the reference's topological sort,
    rt::optimize and ThreadPoolRunner) gives what the operator functions give."""
    import oracle
    N, H, W, C, kh, kw, O, s = 2, 8, 8, 3, 5, 5, 4, 2
    x, k, dy = rand_conv_inputs(11, N, H, W, C, kh, kw, O, s)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    prog = oracle.RefProgram()
    a, y = prog.conv2d(x, k, (s, s), pads)
    b, dx = prog.conv2d_input_grad(dy, k, s, (H, W))
    c, dk = prog.conv2d_kernel_grad(dy, x, s, pads)
    prog.run([a, b, c], mcpu=mcpu, workers=4)
    eq(y, ref.conv2d(x, k, (s, s)))
    eq(dx, ref.conv2d_input_grad(dy, k, s, (H, W)))
    eq(dk, ref.conv2d_kernel_grad(dy, x, s, pads))

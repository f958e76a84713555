"""What the mathematics fixes, for the parts of the oracle that no stored vector covers:
adjoint identities, torch float64 convolution / autograd on DCGAN-shaped (5x5, stride 2, SAME)
cases, the SAME-pad table, and the xorshift stream."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from common import rand_conv_inputs, same_pad

SHAPES = [  # N, H, W, C, kh, kw, O, stride
    (2, 8, 8, 3, 5, 5, 4, 2),
    (1, 16, 16, 8, 5, 5, 16, 2),
    (2, 7, 9, 2, 3, 3, 5, 2),
    (2, 6, 6, 4, 5, 5, 3, 1),
    (1, 9, 7, 2, 3, 5, 2, 3),
]


def torch_conv(x, k, s):
    N, H, W, C = x.shape
    kh, kw, _, O = k.shape
    ph, pw = same_pad(H, kh, s)[0], same_pad(W, kw, s)[0]
    xt = F.pad(x.permute(0, 3, 1, 2), (pw // 2, pw - pw // 2, ph // 2, ph - ph // 2))
    return F.conv2d(xt, k.permute(3, 2, 0, 1), stride=s).permute(0, 2, 3, 1)


@pytest.mark.parametrize("shape", SHAPES)
def test_conv_and_grads_vs_torch_f64(orc, orc64, shape):
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(21, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    kt = torch.tensor(k, dtype=torch.float64, requires_grad=True)
    y = torch_conv(xt, kt, s)
    y.backward(torch.tensor(dy, dtype=torch.float64))
    for o, tol in ((orc, 2e-5), (orc64, 2e-6)):
        np.testing.assert_allclose(o.conv2d(x, k, (s, s)), y.detach().numpy(), rtol=tol, atol=tol)
        np.testing.assert_allclose(o.conv2d_input_grad(dy, k, s, (H, W)), xt.grad.numpy(), rtol=tol, atol=tol)
        np.testing.assert_allclose(o.conv2d_kernel_grad(dy, x, s, pads), kt.grad.numpy(), rtol=tol, atol=tol)


@pytest.mark.parametrize("shape", SHAPES)
def test_adjoint_identities(orc64, shape):
    """<conv(x,k), dy> = <x, dx(dy,k)> = <k, dk(x,dy)>: a wrong index, sign or rotation breaks it."""
    N, H, W, C, kh, kw, O, s = shape
    x, k, dy = rand_conv_inputs(4, *shape)
    pads = (same_pad(H, kh, s)[0], same_pad(W, kw, s)[0])
    lhs = np.vdot(orc64.conv2d(x, k, (s, s)).astype(np.float64), dy)
    a = np.vdot(x.astype(np.float64), orc64.conv2d_input_grad(dy, k, s, (H, W)))
    b = np.vdot(k.astype(np.float64), orc64.conv2d_kernel_grad(dy, x, s, pads))
    assert abs(lhs - a) <= 1e-5 * max(1, abs(lhs))
    assert abs(lhs - b) <= 1e-5 * max(1, abs(lhs))


@pytest.mark.parametrize("shape", [(2, 4, 4, 6, 5, 5, 3, 2), (1, 8, 8, 4, 5, 5, 2, 2), (2, 3, 5, 2, 3, 3, 4, 2)])
def test_transpose_and_grads_vs_torch_f64(orc, shape):
    """conv2d_transpose with TF 'SAME' output size (out = in * stride) and its two gradients
    -- the shapes the reference's CPU functions cannot do -- against torch autograd."""
    N, Hi, Wi, Ci, kh, kw, Co, s = shape
    rng = np.random.default_rng(8)
    x = rng.uniform(-1, 1, (N, Hi, Wi, Ci)).astype(np.float32)
    k = (rng.standard_normal((kh, kw, Co, Ci)) * 0.1).astype(np.float32)
    Ho, Wo = Hi * s, Wi * s
    dy = rng.uniform(-1, 1, (N, Ho, Wo, Co)).astype(np.float32)
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    kt = torch.tensor(k, dtype=torch.float64, requires_grad=True)
    full = F.conv_transpose2d(xt.permute(0, 3, 1, 2), kt.permute(3, 2, 0, 1), stride=s)
    ph, pw = (Hi - 1) * s + kh - Ho, (Wi - 1) * s + kw - Wo
    y = full[:, :, ph // 2:ph // 2 + Ho, pw // 2:pw // 2 + Wo].permute(0, 2, 3, 1)
    y.backward(torch.tensor(dy, dtype=torch.float64))
    np.testing.assert_allclose(orc.conv2d_transpose(x, k, (Ho, Wo), s), y.detach().numpy(), rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(orc.conv2d_transpose_input_grad(dy, k, s, (Hi, Wi)), xt.grad.numpy(), rtol=2e-5, atol=2e-5)
    np.testing.assert_allclose(orc.conv2d_transpose_kernel_grad(dy, x, s, (kh, kw)), kt.grad.numpy(), rtol=2e-5, atol=2e-5)


def test_same_pad_table():
    # DCGAN: every 5x5 stride-2 layer pads (1, 2); the reference literals pad (0,1) and (1,1)
    for n in (64, 32, 16, 8, 4):
        assert same_pad(n, 5, 2) == (3, n // 2)
    assert same_pad(3, 2, 2) == (1, 2)
    assert same_pad(5, 3, 2) == (2, 3)
    assert same_pad(4, 2, 2) == (0, 2)
    assert same_pad(7, 1, 3) == (0, 3)


def test_xorshift_stream():
    """First outputs of the generator, worked by hand from its recurrence in Python integers."""
    import oracle
    s = [1000 * 234, 2000 * 234, 3000 * 234, 4000 * 234]
    M = (1 << 64) - 1
    exp = []
    for _ in range(6):
        t = (s[0] ^ (s[0] << 11)) & M
        s = [s[1], s[2], s[3], (s[3] ^ (s[3] >> 19) ^ t ^ (t >> 8)) & M]
        exp.append(s[3])
    r = oracle.XorShift(234)
    assert [r.next_u64() for _ in range(6)] == exp
    f = oracle.XorShift(234).f32((6,))
    np.testing.assert_array_equal(f, (np.array(exp, dtype=np.float32) / np.float32(M)).astype(np.float32))
    assert (f >= 0).all() and (f <= 1).all()


def test_adam_lrt_closed_form():
    import oracle
    t, lrt = oracle.Oracle.adam_lrt(0, 0.45, 0.68, 0.27)
    assert t == 1 and abs(lrt - 0.45 * np.sqrt(0.73) / 0.32) < 1e-6
    t, lrt = oracle.Oracle.adam_lrt(t, 2e-4, 0.5, 0.999)
    assert t == 2 and abs(lrt - 2e-4 * np.sqrt(1 - 0.999 ** 2) / (1 - 0.25)) < 1e-9

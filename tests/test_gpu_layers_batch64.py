"""The reference's layer-size suite at its own size: batch 64, 5x5 filters, stride 2, SAME padding, the four
discriminator layers (conv2d, its input gradient, its filter gradient) and the four generator layers
(conv2d_transpose and its two gradients), gradients taken through `reshape -> mse` against a random
target as the reference's tests do, inputs and filters standard normal -- reference
tests/test_conv_d0.cu:42-60, test_conv_dx_d0.cu:42-64, test_conv_dk_d0.cu:42-64, test_conv_g0.cu,
test_conv_dk_g0.cu (d1-d3 / g1-g3 alike) -- and the two stacked tests on the seeded xorshift stream,
tests/test_conv_s1.cu:31-77 and test_conv_s2.cu:33-86.

Every result is compared with the CPU oracle twice (common.agree): element by element at 1e-4 relative /
1e-5 absolute, the absolute part widened by the largest magnitude of tensors that exceed 1 (forward
results are sums of thousands of O(1) products), and against the float64-accumulating twin of the
oracle with the oracle's own fp32 rounding error as the yardstick:
max |gpu - f64| <= max(2 * max |oracle32 - f64|, 1e-5 * min(1, max |result|)) -- the check that carries
the mse-wrapped gradients, whose magnitude is 1e-3 to 1e-1.

The input-gradient products (conv2d input gradient, conv2d_transpose forward) get 2 * 3 in place of 2:
the reference adds, per output element, one partial convolution of at most ceil(5/2)^2 = 9 products per
filter to a running sum (src/cpu/ops.hxx:651-672), so its running sum is 9 times shorter than that of a
kernel which adds the same products one after another, and its fp32 error smaller by about sqrt(9).
Measured ratios max |gpu - f64| / max |oracle32 - f64| on MI355X: 0.1-1.2 for forward products and
filter gradients, 0.4-3.5 for the input-gradient products."""
import numpy as np
import pytest

from common import agree, same_pad

pytestmark = pytest.mark.gpu

BATCH = 64
#        name   H   C    O         conv2d: x [BATCH,H,H,C] * w [5,5,C,O] -> [BATCH,H/2,H/2,O]
D_LAYERS = {"d0": (64, 3, 64), "d1": (32, 64, 128), "d2": (16, 128, 256), "d3": (8, 256, 512)}
#        name   Hi  Ci   Co        conv2d_transpose: x [BATCH,Hi,Hi,Ci] * w [5,5,Co,Ci] -> [BATCH,2Hi,2Hi,Co]
G_LAYERS = {"g0": (4, 512, 256), "g1": (8, 256, 128), "g2": (16, 128, 64), "g3": (32, 64, 3)}

_cache = {}


@pytest.fixture(scope="module")
def be():
    import __graft_entry__ as ge
    return ge.load_package().HipBackend(0)


BLOCKED = 3.0   # sqrt(9): see the module docstring


def flat(a):
    return a.reshape(a.shape[0], -1)


def conv_layer(name, orc, orc64):
    """Inputs of one discriminator-layer test and the oracle's results (fp32 and float64 twin)."""
    if name not in _cache:
        H, C, O = D_LAYERS[name]
        rng = np.random.default_rng(sum(map(ord, name)))
        x = rng.standard_normal((BATCH, H, H, C)).astype(np.float32)
        w = rng.standard_normal((5, 5, C, O)).astype(np.float32)
        y = rng.standard_normal((BATCH, H // 2, H // 2, O)).astype(np.float32)
        pads = (same_pad(H, 5, 2)[0],) * 2
        exp = []
        for o in (orc, orc64):
            o.set_threads(16)
            y_hat = o.conv2d(x, w, (2, 2))
            dy = o.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
            exp.append({"y_hat": y_hat, "dy": dy, "dx": o.conv2d_input_grad(dy, w, 2, (H, H)),
                        "dk": o.conv2d_kernel_grad(dy, x, 2, pads, (5, 5))})
        _cache[name] = (x, w, y, pads, exp[0], exp[1])
    return _cache[name]


def transpose_layer(name, orc, orc64):
    if name not in _cache:
        Hi, Ci, Co = G_LAYERS[name]
        rng = np.random.default_rng(sum(map(ord, name)))
        x = rng.standard_normal((BATCH, Hi, Hi, Ci)).astype(np.float32)
        w = rng.standard_normal((5, 5, Co, Ci)).astype(np.float32)
        y = rng.standard_normal((BATCH, 2 * Hi, 2 * Hi, Co)).astype(np.float32)
        exp = []
        for o in (orc, orc64):
            o.set_threads(16)
            y_hat = o.conv2d_transpose(x, w, (2 * Hi, 2 * Hi), 2)
            dy = o.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
            exp.append({"y_hat": y_hat, "dy": dy, "dx": o.conv2d_transpose_input_grad(dy, w, 2, (Hi, Hi)),
                        "dk": o.conv2d_transpose_kernel_grad(dy, x, 2, (5, 5))})
        _cache[name] = (x, w, y, exp[0], exp[1])
    return _cache[name]


@pytest.mark.parametrize("name", list(D_LAYERS))
def test_conv_d(be, orc, orc64, name):
    """conv2d forward of layer d0..d3 (reference tests/test_conv_d0.cu:42-60 and its siblings)."""
    print("layer", name, flush=True)
    x, w, y, pads, e32, e64 = conv_layer(name, orc, orc64)
    agree(be.conv2d(x, w, (2, 2)), e32["y_hat"], e64["y_hat"], name + " conv2d")


@pytest.mark.parametrize("name", list(D_LAYERS))
def test_conv_dx_d(be, orc, orc64, name):
    """d mse(y, conv2d(x, w)) / dx (reference tests/test_conv_dx_d0.cu:42-64)."""
    print("layer", name, flush=True)
    x, w, y, pads, e32, e64 = conv_layer(name, orc, orc64)
    H = x.shape[1]
    y_hat = be.conv2d(x, w, (2, 2))
    dy = be.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
    agree(dy, e32["dy"], e64["dy"], name + " mse gradient")
    agree(be.conv2d_input_grad(dy, w, 2, (H, H)), e32["dx"], e64["dx"], name + " conv2d input gradient", BLOCKED)


@pytest.mark.parametrize("name", list(D_LAYERS))
def test_conv_dk_d(be, orc, orc64, name):
    """d mse(y, conv2d(x, w)) / dw (reference tests/test_conv_dk_d0.cu:42-64)."""
    print("layer", name, flush=True)
    x, w, y, pads, e32, e64 = conv_layer(name, orc, orc64)
    y_hat = be.conv2d(x, w, (2, 2))
    dy = be.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
    agree(be.conv2d_kernel_grad(dy, x, 2, pads, (5, 5)), e32["dk"], e64["dk"], name + " conv2d filter gradient")


@pytest.mark.parametrize("name", list(G_LAYERS))
def test_conv_g(be, orc, orc64, name):
    """conv2d_transpose forward of layer g0..g3 (reference tests/test_conv_g0.cu)."""
    print("layer", name, flush=True)
    x, w, y, e32, e64 = transpose_layer(name, orc, orc64)
    Ho = 2 * x.shape[1]
    agree(be.conv2d_transpose(x, w, (Ho, Ho), 2), e32["y_hat"], e64["y_hat"], name + " conv2d_transpose", BLOCKED)


@pytest.mark.parametrize("name", list(G_LAYERS))
def test_conv_dx_g(be, orc, orc64, name):
    """d mse(y, conv2d_transpose(x, w)) / dx (reference tests/ref_conv_dx_g0.py:13-23)."""
    print("layer", name, flush=True)
    x, w, y, e32, e64 = transpose_layer(name, orc, orc64)
    Hi = x.shape[1]
    y_hat = be.conv2d_transpose(x, w, (2 * Hi, 2 * Hi), 2)
    dy = be.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
    agree(be.conv2d_transpose_input_grad(dy, w, 2, (Hi, Hi)), e32["dx"], e64["dx"], name + " transpose input gradient")


@pytest.mark.parametrize("name", list(G_LAYERS))
def test_conv_dk_g(be, orc, orc64, name):
    """d mse(y, conv2d_transpose(x, w)) / dw (reference tests/test_conv_dk_g0.cu)."""
    print("layer", name, flush=True)
    x, w, y, e32, e64 = transpose_layer(name, orc, orc64)
    Hi = x.shape[1]
    y_hat = be.conv2d_transpose(x, w, (2 * Hi, 2 * Hi), 2)
    dy = be.mse_grad(flat(y), flat(y_hat)).reshape(y_hat.shape)
    agree(be.conv2d_transpose_kernel_grad(dy, x, 2, (5, 5)), e32["dk"], e64["dk"], name + " transpose filter gradient")


@pytest.mark.parametrize("name", list(D_LAYERS))
def test_paired_launches_d(be, orc, orc64, name):
    """The two discriminator towers of the training iteration share their filters and run as paired
    launches at batch 64: the layer's inputs as one instance, the same tensors in reversed image order
    as the other, so that each instance must reproduce the oracle's result (reversed for the second)
    and the paired filter gradient is the oracle's gradient twice."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    print("layer", name, flush=True)
    x, w, y, pads, e32, e64 = conv_layer(name, orc, orc64)
    H, C, O = D_LAYERS[name]
    x2 = np.ascontiguousarray(x[::-1])
    dy, dy2 = e32["dy"], np.ascontiguousarray(e32["dy"][::-1])
    if C % 16 == 0:
        y1, y2 = be.conv2d_pair(x, x2, w, (2, 2))
        agree(y1, e32["y_hat"], e64["y_hat"], name + " paired forward, first instance")
        agree(y2[::-1], e32["y_hat"], e64["y_hat"], name + " paired forward, second instance")
        g1, g2 = be.conv2d_input_grad_pair(dy, dy2, w, 2, (H, H))
        agree(g1, e32["dx"], e64["dx"], name + " paired input gradient, first instance", BLOCKED)
        agree(g2[::-1], e32["dx"], e64["dx"], name + " paired input gradient, second instance", BLOCKED)
    else:
        assert A.load().dh_conv2d_dk_pair_supported(BATCH, H, H, C, H // 2, H // 2, O, 5, 5, 2, 2) == 1
    agree(be.conv2d_kernel_grad_pair(dy, x, dy2, x2, 2, pads), 2 * e32["dk"], 2 * e64["dk"], name + " paired filter gradient")


def stacked_inputs():
    """xorshift stream, seed 234, in the order the reference's stacked tests draw it."""
    import oracle
    gen = oracle.XorShift(234)
    x = gen.f32((BATCH, 64, 64, 3))
    ws = [gen.f32((5, 5, c, o)) for c, o in ((3, 64), (64, 128), (128, 256), (256, 512))]
    y = gen.f32((BATCH, 4 * 4 * 512))
    return x, ws, y


def test_conv_s1(be, orc, orc64):
    """Four stacked conv2d layers, forward (reference tests/test_conv_s1.cu:31-77)."""
    x, ws, _ = stacked_inputs()
    got, e32, e64 = x, x, x
    orc.set_threads(16), orc64.set_threads(16)
    for i, w in enumerate(ws):
        got, e32, e64 = be.conv2d(got, w, (2, 2)), orc.conv2d(e32, w, (2, 2)), orc64.conv2d(e64, w, (2, 2))
        agree(got, e32, e64, "stacked forward, layer %d" % i)
    assert got.shape == (BATCH, 4, 4, 512)


def test_conv_s2(be, orc, orc64):
    """Gradient of mse(y, four stacked conv2d layers) with respect to the images
    (reference tests/test_conv_s2.cu:33-86)."""
    x, ws, y = stacked_inputs()
    orc.set_threads(16), orc64.set_threads(16)
    res = []
    for o in (be, orc, orc64):
        acts = [x]
        for w in ws:
            acts.append(o.conv2d(acts[-1], w, (2, 2)))
        g = o.mse_grad(y, flat(acts[-1])).reshape(acts[-1].shape)
        for w, a in zip(ws[::-1], acts[-2::-1]):
            g = o.conv2d_input_grad(g, w, 2, a.shape[1:3])
        res.append(g)
    assert res[0].shape == x.shape
    agree(res[0], res[1], res[2], "stacked input gradient", BLOCKED)

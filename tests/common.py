"""Helpers shared by the oracle tests (CPU) and the parity tests (GPU).

`run_case(be, case)` replays one golden case -- the literal inputs of one of the reference's own
operator tests -- through a backend `be` that offers the operator methods of `oracle.Oracle`
(the HIP front-end offers the same ones) and returns the tensors the reference test exports.
"""
import numpy as np

# north_star tolerance for fp32 results: 1e-4 relative / 1e-5 absolute
RTOL, ATOL = 1e-4, 1e-5


def agree(got, exp32, exp64, what, slack=1.0, elementwise=True, kinks=0, kink_extra=0.0):
    """The two-sided parity check of the batch-64 suites.  `exp32` is the oracle's fp32 result (the
    reference's arithmetic and summation order), `exp64` the same computed with float64 sums.
      * element by element: |got - exp32| <= 1e-4 |exp32| + max(1e-5 max(1, max|exp32|), 3 max|exp32 - exp64|)
        -- the stated fp32 tolerance, its absolute part widened for tensors of large magnitude (sums of
        thousands of O(1) products cannot be held to 1e-5 by any fp32 summation order) and never below
        three times the oracle's OWN distance from the float64 result: the reference's serial fp32 sum
        over 65 536 rows (the first layer's bias gradient) is itself 1.4e-5 away from the exact sum, and
        a result that is 3e-8 from exact must not fail for disagreeing with it;
      * against the float64 result, with the oracle's own fp32 rounding error as the yardstick:
        max |got - exp64| <= max(2 * slack * max |exp32 - exp64|, 1e-5 * min(1, max|exp32|)) -- the
        floor follows the magnitude downwards, so that gradients of magnitude 1e-6 are not waved
        through by an absolute 1e-5.
    slack = 3 for results downstream of an input-gradient product: there the reference adds blocks of
    up to ceil(5/2)^2 = 9 products to its running sum (src/cpu/ops.hxx:651-672), which makes its fp32
    error about sqrt(9) smaller than that of a kernel adding the same products one by one.
    kinks: the tensor is a gradient through relu / leaky-relu layers.  A pre-activation within rounding
    distance of zero takes either slope, depending on the summation order that produced it, and the
    gradients downstream then differ by that element's whole contribution (measured between the batch-64
    and the batch-512 kernels on the same images: 1 element of 4 194 304 in one generator layer, 1 of
    2 097 152 in another, none elsewhere -- and three bias / filter gradients off by 1.4e-4 to 3.9e-4 of
    their largest value in single entries; and between two summation orders of the batch-64 kernels: one
    output of the third discriminator layer is -1.9e-10 on the GPU, +4.0e-8 in the oracle's fp32 run and
    +4.4e-8 in float64, and entry 16 of that layer's bias gradient, 0.0348, moves by 5.7e-5 = 0.8 times the
    gradient arriving there; the eight entries of that layer's filter gradient that meet the largest inputs
    move by up to 1.35e-5 = 2.3e-3 of the tensor's largest entry).  A caller sets `kinks` only where it has
    FOUND such elements, and passes their number (the DCGAN tests look for layer outputs of opposite sign at the
    rounding level and count those the gradient flows back through).  Such tensors are allowed 5e-3 of their
    largest magnitude in the float64 check, their relative L2 error is held to 1e-3, and in the
    element-by-element check one entry per kink (one per 100 000 entries and kink for larger tensors: a flipped
    slope reaches a whole filter column) may be off by up to that 5e-3 as well.  kink_extra is added to that
    allowance where the caller can bound the flipped slope's direct effect from the data (the filter gradient of
    the kinked layer itself moves by input patch x the change of the layer's bias gradient)."""
    got, exp32, exp64 = (np.asarray(a, np.float64).reshape(-1) for a in (got, exp32, exp64))
    mag = float(np.abs(exp32).max()) if exp32.size else 0.0
    yard = float(np.abs(exp32 - exp64).max()) if exp32.size else 0.0
    err = float(np.abs(got - exp64).max()) if exp32.size else 0.0
    print("%-50s max|exp| %.3g  oracle32-f64 %.3g  gpu-f64 %.3g  ratio %.2f" % (what, mag, yard, err, err / max(yard, 1e-30)),
          flush=True)
    if elementwise:
        atol = max(ATOL * max(1.0, mag), 3.0 * yard)
        over = np.abs(got - exp32) > atol + RTOL * np.abs(exp32)
        # a kink shows in single entries (see above): they are held to the float64 check's 5e-3 instead
        few = kinks and 0 < int(over.sum()) <= int(kinks) * max(1, exp32.size // 100000) and \
            float(np.abs(got - exp32)[over].max()) <= 5e-3 * mag + kink_extra
        if few:
            print("%-50s %d entr%s at a kink: off by %.3g" % (what, int(over.sum()), "y" if over.sum() == 1 else "ies",
                                                              float(np.abs(got - exp32)[over].max())), flush=True)
        else:
            np.testing.assert_allclose(got, exp32, rtol=RTOL, atol=atol, err_msg=what)
    if kinks and exp32.size:
        l2 = float(np.linalg.norm(got - exp64) / max(np.linalg.norm(exp64), 1e-30))
        assert l2 <= 1e-3, "%s: relative L2 error %.3g" % (what, l2)
    assert err <= max(2.0 * slack * yard, ATOL * min(1.0, mag), 5e-3 * mag + kink_extra if kinks else 0.0), \
        "%s: max |gpu - f64| = %.3g, the oracle's own fp32 error is %.3g (max |exp| = %.3g)" % (what, err, yard, mag)


def get(case, key, kind="inputs"):
    a = case[kind][key]
    return np.array(a["data"], dtype=np.float64).reshape(a["shape"])


def same_pad(n_in, k, s):
    p = k - s if n_in % s == 0 else k - (n_in % s)
    return max(p, 0), -(-n_in // s)


def mse_dy(be, y, y_hat):
    """Gradient of the reference tests' `reshape -> mse` wrapper w.r.t. y_hat
    (reference: src/cpu/kernels.cu:110-113)."""
    return be.mse_grad(y.reshape(y.shape[0], -1), y_hat.reshape(y.shape[0], -1)).reshape(y_hat.shape)


def run_case(be, case):
    op, p = case["op"], case["params"]
    I = lambda k: get(case, k).astype(np.float32)
    if op == "conv2d":
        return {"y": be.conv2d(I("x"), I("k"), p["strides"])}
    if op == "conv2d_grad":
        x, k, y = I("x"), I("k"), I("y")
        s = p["strides"]
        pads = (same_pad(x.shape[1], k.shape[0], s[0])[0], same_pad(x.shape[2], k.shape[1], s[1])[0])
        y_hat = be.conv2d(x, k, s)
        dy = mse_dy(be, y, y_hat)
        return {"y_hat": y_hat, "dy_hat": dy,
                "dx": be.conv2d_input_grad(dy, k, s[0], x.shape[1:3]),
                "dk": be.conv2d_kernel_grad(dy, x, s[0], pads, k.shape[:2]),
                "loss": be.mse(y.reshape(y.shape[0], -1), y_hat.reshape(y.shape[0], -1))}
    if op == "conv2d_transpose":
        return {"y": be.conv2d_transpose(I("x"), I("k"), p["out_size"][1:3], p["strides"][0])}
    if op == "conv2d_transpose_grad":
        x, k, y = I("x"), I("k"), I("y")
        s = p["strides"][0]
        y_hat = be.conv2d_transpose(x, k, p["out_size"][1:3], s)
        dy = mse_dy(be, y, y_hat)
        return {"y_hat": y_hat, "dy_hat": dy,
                "dx": be.conv2d_transpose_input_grad(dy, k, s, x.shape[1:3]),
                "dk": be.conv2d_transpose_kernel_grad(dy, x, s, k.shape[:2]),
                "loss": be.mse(y.reshape(y.shape[0], -1), y_hat.reshape(y.shape[0], -1))}
    if op == "bias_add":
        return {"out": be.bias_add(I("z"), I("b"))}
    if op == "bias_add_grad":
        z, b, y = I("z"), I("b"), I("y")
        dy = mse_dy(be, y, be.bias_add(z, b))
        return {"dy_hat": dy, "dx": dy, "db": be.bias_grad(dy)}
    if op == "mat_sum_cols":
        return {"out": be.bias_grad(I("x"))}
    if op == "relu_leaky":
        return {"out": be.relu_leaky(I("x"), p["alpha"])}
    if op in ("relu", "tanh", "sigmoid"):
        return {"out": getattr(be, op)(I("x"))}
    if op in ("leaky_relu_grad", "relu_grad", "tanh_grad", "sigmoid_grad"):
        x, y = I("x"), I("y")
        fwd = {"leaky_relu_grad": lambda v: be.relu_leaky(v, p["alpha"]), "relu_grad": be.relu,
               "tanh_grad": be.tanh, "sigmoid_grad": be.sigmoid}[op]
        y_hat = fwd(x)
        dy = mse_dy(be, y, y_hat)
        if op == "leaky_relu_grad":
            dx = be.leaky_relu_grad(x, dy, p["alpha"])
        elif op == "relu_grad":
            dx = be.relu_grad(x, dy)
        else:  # tanh / sigmoid gradients take the forward OUTPUT
            dx = getattr(be, op)(y_hat, dy)
        return {"y_hat": y_hat, "dy_hat": dy, "dx": dx}
    if op == "add":
        return {"out": be.add(I("a"), I("b"))}
    if op == "argmax_acc":
        return {"acc": np.array(float(be.argmax_acc(I("y"), I("y_hat"))))}
    if op == "sigmoid_cross_entropy":
        x, y = I("x"), I("y")
        return {"loss": np.array(be.sigmoid_cross_entropy(y.reshape(-1), x.reshape(-1))),
                "dx": be.sigmoid_cross_entropy_grad(y, x)}
    if op == "moment_update":
        return {"out": be.moment_update(I("var"), I("dv"), p["c1"], p["c2"])}
    if op == "moment_update2":
        return {"out": be.moment_update2(I("var"), I("dv"), p["c1"], p["c2"])}
    if op == "adam_update":
        t, lrt = be.adam_lrt(p["t_before"], p["lr"], p["beta1"], p["beta2"])
        assert t == 1.0
        return {"out": be.adam_apply(I("x"), I("m"), I("v"), lrt, p["eps"])}
    if op == "mat_mul_add":
        return {"out": be.mat_mul_add(I("x"), I("w"), I("b"))}
    if op in ("mm_mul", "tmm_mul", "mtm_mul"):
        return {"out": getattr(be, op)(I("a"), I("b"))}
    raise KeyError(op)


def check_case(be, case, rtol=RTOL, atol=ATOL):
    got = run_case(be, case)
    for key, exp in case["expected"].items():
        e = np.array(exp["data"], dtype=np.float64).reshape(exp["shape"])
        g = np.asarray(got[key], dtype=np.float64).reshape(e.shape)
        np.testing.assert_allclose(g, e, rtol=rtol, atol=atol,
                                   err_msg="%s / %s (%s)" % (case["name"], key, case["source"]))


GOLDEN_NAMES = [
    "conv2d", "conv2d_padding", "conv2d_grad", "conv2d_padding_grad", "conv2d_transpose",
    "conv2d_transpose_grad", "conv2d_bias_add", "conv2d_bias_add_grad", "vect_relu_leaky",
    "vect_relu", "vect_tanh", "sigmoid", "leaky_relu_grad", "relu_grad", "tanh_grad",
    "sigmoid_grad", "add", "argmax_accuracy", "sigmoid_cross_entropy", "moment_update",
    "moment_update2", "adam_update", "mat_mul_add", "mat_mat_mul", "tmat_mat_mul",
    "mat_tmat_mul", "mat_rvect_add", "mat_sum_cols"]


def rand_conv_inputs(seed, N, H, W, C, kh, kw, O, s):
    """Seeded inputs in the distributions the benchmark configurations name:
    x ~ U(-1,1), k ~ N(0, 0.02), dy ~ U(-1,1)."""
    rng = np.random.default_rng(seed)
    x = rng.uniform(-1, 1, (N, H, W, C)).astype(np.float32)
    k = (rng.standard_normal((kh, kw, C, O)) * 0.02).astype(np.float32)
    Ho, Wo = -(-H // s), -(-W // s)
    dy = rng.uniform(-1, 1, (N, Ho, Wo, O)).astype(np.float32)
    return x, k, dy

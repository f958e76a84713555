"""Bias, activation, loss, dense and Adam kernels against the CPU oracle at sizes that cover the
vector path, the scalar tail, the narrow (3-channel) and wide (512 / 8192 column) reductions."""
import numpy as np
import pytest

from common import RTOL, ATOL

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def be():
    import __graft_entry__ as ge
    return ge.load_package().HipBackend(0)


def close(got, exp, scale=1.0):
    np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL * scale)


# 8389635 floats: past the size from which the maps run one 16-byte access per thread instead of a
# capped grid-stride loop (8192 workgroups), with a scalar tail
@pytest.mark.parametrize("n", [1, 3, 255, 1024, 4099, 786432, 8389635])
def test_activations_and_grads(be, orc, n):
    rng = np.random.default_rng(n)
    a = rng.uniform(-4, 4, n).astype(np.float32)
    d = rng.uniform(-1, 1, n).astype(np.float32)
    a[:1] = 0.0
    np.testing.assert_array_equal(be.relu(a), orc.relu(a))
    np.testing.assert_array_equal(be.relu_leaky(a, 0.2), orc.relu_leaky(a, 0.2))
    np.testing.assert_array_equal(be.relu_grad(a, d), orc.relu_grad(a, d))
    np.testing.assert_array_equal(be.leaky_relu_grad(a, d, 0.2), orc.leaky_relu_grad(a, d, 0.2))
    close(be.tanh(a), orc.tanh(a))
    close(be.sigmoid(a), orc.sigmoid(a))
    t, s = orc.tanh(a), orc.sigmoid(a)
    close(be.tanh_grad(t, d), orc.tanh_grad(t, d))
    close(be.sigmoid_grad(s, d), orc.sigmoid_grad(s, d))
    np.testing.assert_array_equal(be.add(a, d), orc.add(a, d))


@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 3), (64, 1), (4096, 3), (1000, 64), (333, 128), (64, 512), (64, 8192), (5, 300), (4097, 20),
                                       (131073, 64)])
def test_bias_add_and_grad(be, orc, rows, cols):
    rng = np.random.default_rng(rows * 31 + cols)
    z = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    b = rng.standard_normal(cols).astype(np.float32)
    np.testing.assert_array_equal(be.bias_add(z, b), orc.bias_add(z, b))
    exp = orc.bias_grad(z)
    close(be.bias_grad(z), exp, scale=max(1.0, np.sqrt(rows)))
    close(be.mat_sum_rows(z), orc.mat_sum_rows(z), scale=max(1.0, np.sqrt(cols)))


@pytest.mark.parametrize("act", ["relu", "leaky", "tanh", "none"])
@pytest.mark.parametrize("rows,cols", [(2048, 64), (1031, 3), (64, 512)])
def test_fused_act_bias_grad(be, orc, act, rows, cols):
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    rng = np.random.default_rng(7)
    z = rng.uniform(-2, 2, (rows, cols)).astype(np.float32)
    d = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    if act == "relu":
        ref, dz, code = orc.relu(z), orc.relu_grad(z, d), A.ACT_RELU          # forward OUTPUT as reference
    elif act == "leaky":
        ref, dz, code = orc.relu_leaky(z, 0.2), orc.leaky_relu_grad(z, d, 0.2), A.ACT_LEAKY
    elif act == "tanh":
        ref = orc.tanh(z)
        dz, code = orc.tanh_grad(ref, d), A.ACT_TANH
    else:
        ref, dz, code = z, d, A.ACT_NONE
    got_dz, got_db = be.act_bias_grad(ref, d, code, 0.2)
    close(got_dz, dz)
    close(got_db, orc.bias_grad(dz), scale=max(1.0, np.sqrt(rows)))


def test_losses(be, orc):
    rng = np.random.default_rng(2)
    for n in (1, 64, 512, 5000):
        x = rng.uniform(-6, 6, n).astype(np.float32)
        y = (rng.uniform(0, 1, n) > 0.5).astype(np.float32)
        close(be.sigmoid_cross_entropy(y, x), orc.sigmoid_cross_entropy(y, x))
        close(be.sigmoid_cross_entropy_grad(y, x), orc.sigmoid_cross_entropy_grad(y, x))
    a = rng.uniform(-1, 1, (16, 40)).astype(np.float32)
    b = rng.uniform(-1, 1, (16, 40)).astype(np.float32)
    close(be.mse(a, b), orc.mse(a, b))
    close(be.mse_grad(a, b), orc.mse_grad(a, b))


def test_loss_and_gradient_in_one_launch(be, orc):
    """dh_sigmoid_cross_entropy_head: loss and gradient of one or two logit vectors and the sum of two losses
    are the values of the separate entry points to the bit."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    rng = np.random.default_rng(21)
    for n in (1, 64, 512, 5000):
        print("n", n, flush=True)
        xs = [rng.uniform(-6, 6, n).astype(np.float32) for _ in range(2)]
        ys = [(rng.uniform(0, 1, n) > 0.5).astype(np.float32) for _ in range(2)]
        sep_loss = [be.sigmoid_cross_entropy(y, x) for y, x in zip(ys, xs)]
        sep_grad = [be.sigmoid_cross_entropy_grad(y, x) for y, x in zip(ys, xs)]
        dy, dx = [A.Buf.from_numpy(y) for y in ys], [A.Buf.from_numpy(x) for x in xs]
        loss, grad, total = [A.Buf((1,)) for _ in range(2)], [A.Buf((n,)) for _ in range(2)], A.Buf((1,))
        A.check(lib.dh_sigmoid_cross_entropy_head(dy[0].ptr, dx[0].ptr, loss[0].ptr, grad[0].ptr, dy[1].ptr, dx[1].ptr,
                                                  loss[1].ptr, grad[1].ptr, total.ptr, n, None))
        for q in range(2):
            np.testing.assert_array_equal(loss[q].numpy()[0], np.float32(sep_loss[q]))
            np.testing.assert_array_equal(grad[q].numpy(), sep_grad[q])
        np.testing.assert_array_equal(total.numpy()[0], np.float32(sep_loss[0]) + np.float32(sep_loss[1]))
        close(grad[0].numpy(), orc.sigmoid_cross_entropy_grad(ys[0], xs[0]))
        # one vector, gradient only / loss only
        g1, l1 = A.Buf((n,)), A.Buf((1,))
        A.check(lib.dh_sigmoid_cross_entropy_head(dy[1].ptr, dx[1].ptr, None, g1.ptr, None, None, None, None, None, n, None))
        A.check(lib.dh_sigmoid_cross_entropy_head(dy[1].ptr, dx[1].ptr, l1.ptr, None, None, None, None, None, None, n, None))
        np.testing.assert_array_equal(g1.numpy(), sep_grad[1])
        np.testing.assert_array_equal(l1.numpy()[0], np.float32(sep_loss[1]))
    with pytest.raises(A.HipError, match="two logit vectors"):
        A.check(lib.dh_sigmoid_cross_entropy_head(dy[0].ptr, dx[0].ptr, loss[0].ptr, None, None, None, None, None, total.ptr,
                                                  n, None))


@pytest.mark.parametrize("m,n,p", [(64, 100, 8192), (64, 8192, 1), (9, 33, 17), (1, 64, 8192), (130, 70, 65)])
def test_dense_with_activation_in_the_write_out(be, orc, m, n, p):
    """dh_gemm_nn_act = dh_gemm_nn followed by the activation, to the bit (every kernel the shapes route to)."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    rng = np.random.default_rng(m * 3 + n + p)
    x = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    w = (rng.standard_normal((n, p)) * 0.05).astype(np.float32)
    b = rng.standard_normal(p).astype(np.float32) * 0.1
    z = be.mat_mul_add(x, w, b)
    dx, dw, db, out = A.Buf.from_numpy(x), A.Buf.from_numpy(w), A.Buf.from_numpy(b), A.Buf((m, p))
    for act, alpha, ref in ((A.ACT_RELU, 0.0, np.maximum(z, 0)), (A.ACT_LEAKY, 0.2, be.relu_leaky(z, 0.2)),
                            (A.ACT_NONE, 0.0, z)):
        A.check(lib.dh_gemm_nn_act(dx.ptr, dw.ptr, db.ptr, out.ptr, m, n, p, act, alpha, None))
        np.testing.assert_array_equal(out.numpy(), ref)
    orc.set_threads(8)
    close(np.maximum(z, 0), orc.relu(orc.mat_mul_add(x, w, b)))


@pytest.mark.parametrize("m,n", [(8192, 64), (64, 64), (1000, 37), (200, 1)])
def test_two_dense_weight_gradients_as_one_contraction(be, orc, m, n):
    """dh_gemm_tn_pair: tr(a1) b1 + tr(a2) b2 for a single output column."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    rng = np.random.default_rng(m + n)
    a = [rng.uniform(-1, 1, (n, m)).astype(np.float32) for _ in range(2)]
    g = [rng.uniform(-1, 1, (n, 1)).astype(np.float32) for _ in range(2)]
    assert lib.dh_gemm_tn_pair_supported(m, n, 1) == 1
    da, dg, out = [A.Buf.from_numpy(v) for v in a], [A.Buf.from_numpy(v) for v in g], A.Buf((m, 1))
    A.check(lib.dh_gemm_tn_pair(da[0].ptr, dg[0].ptr, da[1].ptr, dg[1].ptr, out.ptr, m, n, 1, None))
    exp = orc.add(orc.tmm_mul(a[0], g[0]), orc.tmm_mul(a[1], g[1]))
    close(out.numpy(), exp, scale=4)
    exp64 = a[0].astype(np.float64).T @ g[0].astype(np.float64) + a[1].astype(np.float64).T @ g[1].astype(np.float64)
    assert np.abs(out.numpy() - exp64).max() <= 2 * max(np.abs(exp - exp64).max(), 1e-6)
    assert lib.dh_gemm_tn_pair_supported(m, n, 2) == 0 and lib.dh_gemm_tn_pair_supported(m, 65, 1) == 0
    with pytest.raises(A.HipError):
        A.check(lib.dh_gemm_tn_pair(da[0].ptr, dg[0].ptr, da[1].ptr, dg[1].ptr, out.ptr, m, n, 2, None))


def test_argmax_is_exact(be, orc):
    rng = np.random.default_rng(4)
    for rows, cols in ((10, 3), (64, 10), (1500, 7), (3, 1)):
        y = rng.uniform(0, 1, (rows, cols)).astype(np.float32)
        yh = rng.uniform(0, 1, (rows, cols)).astype(np.float32)
        yh[::2] = y[::2]
        y[1, :] = 0.5   # ties -> lowest index on both sides
        assert be.argmax_acc(y, yh) == orc.argmax_acc(y, yh)


# (1, n, p) and (m, n, 1): a vector times a matrix, contraction cut over four wavefronts (whole sixteens, a ragged
# last quarter, fewer rows than wavefronts)
@pytest.mark.parametrize("m,n,p", [(64, 100, 8192), (64, 8192, 1), (9, 33, 17), (1, 1, 1), (130, 70, 65), (64, 128, 200), (3, 5, 64),
                                   (200, 129, 70), (1, 64, 8192), (1, 37, 100), (1, 128, 65), (1, 3, 64), (37, 200, 1),
                                   (128, 64, 1)])
def test_dense(be, orc, m, n, p):
    rng = np.random.default_rng(m + n + p)
    x = rng.uniform(-1, 1, (m, n)).astype(np.float32)
    w = (rng.standard_normal((n, p)) * 0.02).astype(np.float32)
    b = rng.standard_normal(p).astype(np.float32)
    g = rng.uniform(-1, 1, (m, p)).astype(np.float32)
    orc.set_threads(8)
    close(be.mat_mul_add(x, w, b), orc.mat_mul_add(x, w, b))
    close(be.mm_mul(x, w), orc.mm_mul(x, w))
    close(be.tmm_mul(x, g), orc.tmm_mul(x, g), scale=4)    # tr(x) g : dW
    close(be.mtm_mul(g, w), orc.mtm_mul(g, w))             # g tr(w) : dx


@pytest.mark.parametrize("n", [1, 1000, 4099, 3276800, 8389635])
def test_adam(be, orc, n):
    rng = np.random.default_rng(n)
    p = rng.standard_normal(n).astype(np.float32)
    g = rng.standard_normal(n).astype(np.float32)
    m = rng.standard_normal(n).astype(np.float32) * 0.1
    v = rng.uniform(0, 1, n).astype(np.float32) * 0.01
    em, ev = orc.moment_update(m, g, 0.5, 0.5), orc.moment_update2(v, g, 0.999, 0.001)
    close(be.moment_update(m, g, 0.5, 0.5), em)
    close(be.moment_update2(v, g, 0.999, 0.001), ev)
    t, lrt = orc.adam_lrt(0, 2e-4, 0.5, 0.999)
    ep = orc.adam_apply(p, em, ev, lrt, 1e-8)
    close(be.adam_apply(p, em, ev, lrt, 1e-8), ep)
    # the fused single-pass step equals the three separate operators
    gp, gm, gv = be.adam_step(p, m, v, g, 0.5, 0.999, lrt, 1e-8)
    close(gm, em), close(gv, ev), close(gp, ep)
    close(be.vect_update(p, g, -0.1), orc.vect_update(p, g, -0.1))


def test_adam_many_variables_in_one_launch(be, orc):
    """dh_adam_step_multi == the reference's add + moment_update + moment_update2 + adam_update per
    variable: sizes from one element to several workgroups, with and without a second gradient,
    more items than one launch holds, each with its own step size."""
    rng = np.random.default_rng(77)
    sizes = [1, 3, 64, 100, 4095, 4096, 4097, 12800, 204801] + [5 + 7 * i for i in range(20)]
    items, expect = [], []
    for i, n in enumerate(sizes):
        p = rng.standard_normal(n).astype(np.float32)
        g1 = rng.standard_normal(n).astype(np.float32)
        g2 = rng.standard_normal(n).astype(np.float32) if i % 2 == 0 else None
        m = rng.standard_normal(n).astype(np.float32) * 0.1
        v = rng.uniform(0, 1, n).astype(np.float32) * 0.01
        t, lrt = orc.adam_lrt(i % 5, 2e-4, 0.5, 0.999)
        g = orc.add(g1, g2) if g2 is not None else g1
        em, ev = orc.moment_update(m, g, 0.5, 0.5), orc.moment_update2(v, g, 0.999, 0.001)
        expect.append((orc.adam_apply(p, em, ev, lrt, 1e-8), em, ev))
        items.append((p, m, v, g1, g2, lrt))
    got = be.adam_step_multi(items, 0.5, 0.999, 1e-8)
    for (gp, gm, gv), (ep, em, ev) in zip(got, expect):
        close(gm, em), close(gv, ev), close(gp, ep)


def test_empty_inputs(be):
    """Zero-length tensors: the element-wise, bias, dense and Adam entry points return success and
    write nothing; the losses and argmax, whose result divides by the element count, refuse them;
    a null tensor with a non-zero length is refused everywhere."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = be.lib
    guard = np.arange(8, dtype=np.float32) + 1
    buf, src = A.Buf.from_numpy(guard), A.Buf.from_numpy(guard)
    ok = lambda rc: A.check(rc)
    for fn in (lib.dh_relu, lib.dh_tanh, lib.dh_sigmoid):
        ok(fn(src.ptr, buf.ptr, 0, None))
    ok(lib.dh_relu_leaky(src.ptr, buf.ptr, 0, 0.2, None))
    for fn in (lib.dh_relu_grad, lib.dh_tanh_grad, lib.dh_sigmoid_grad, lib.dh_add, lib.dh_mse_grad,
               lib.dh_sigmoid_cross_entropy_grad):
        ok(fn(src.ptr, src.ptr, buf.ptr, 0, None))
    ok(lib.dh_leaky_relu_grad(src.ptr, src.ptr, buf.ptr, 0.2, 0, None))
    ok(lib.dh_bias_add(src.ptr, src.ptr, buf.ptr, 0, 8, None))
    ok(lib.dh_bias_add(src.ptr, src.ptr, buf.ptr, 8, 0, None))
    ok(lib.dh_bias_grad(src.ptr, buf.ptr, 8, 0, None))
    ok(lib.dh_mat_sum_rows(src.ptr, buf.ptr, 0, 8, None))
    ok(lib.dh_gemm_nn(src.ptr, src.ptr, None, buf.ptr, 0, 4, 2, None))
    ok(lib.dh_gemm_tn(src.ptr, src.ptr, buf.ptr, 2, 4, 0, None))
    ok(lib.dh_moment_update(buf.ptr, src.ptr, 0.5, 0.5, 0, None))
    ok(lib.dh_moment_update2(buf.ptr, src.ptr, 0.5, 0.5, 0, None))
    ok(lib.dh_adam_update(buf.ptr, src.ptr, src.ptr, 0.1, 1e-8, 0, None))
    ok(lib.dh_adam_step(buf.ptr, buf.ptr, buf.ptr, src.ptr, 0.5, 0.5, 0.9, 0.1, 0.1, 1e-8, 0, None))
    ok(lib.dh_adam_step_multi(None, 0, 0.5, 0.5, 0.9, 0.1, 1e-8, None))
    item = (A.AdamItem * 1)()
    item[0].p = item[0].m = item[0].v = buf.ptr
    item[0].g1, item[0].g2, item[0].n, item[0].lrt = src.ptr, None, 0, 0.1
    ok(lib.dh_adam_step_multi(item, 1, 0.5, 0.5, 0.9, 0.1, 1e-8, None))
    ok(lib.dh_memset0(buf.ptr, 0, None))
    ok(lib.dh_stream_sync(None))
    np.testing.assert_array_equal(buf.numpy(), guard)
    # the column sum of a matrix without rows is the zero vector; a product over an empty inner
    # extent is the bias (or zero)
    ok(lib.dh_bias_grad(src.ptr, buf.ptr, 0, 8, None))
    np.testing.assert_array_equal(buf.numpy(), np.zeros(8, np.float32))
    buf.write(guard)
    ok(lib.dh_gemm_nn(src.ptr, src.ptr, src.ptr, buf.ptr, 2, 0, 4, None))
    np.testing.assert_array_equal(buf.numpy(), np.concatenate([guard[:4], guard[:4]]))
    ok(lib.dh_gemm_nn(src.ptr, src.ptr, None, buf.ptr, 2, 0, 4, None))
    np.testing.assert_array_equal(buf.numpy(), np.zeros(8, np.float32))
    for bad in (lambda: lib.dh_sigmoid_cross_entropy(src.ptr, src.ptr, buf.ptr, 0, None),
                lambda: lib.dh_mse(src.ptr, src.ptr, buf.ptr, 0, 4, None),
                lambda: lib.dh_argmax_acc(src.ptr, src.ptr, buf.ptr, 4, 0, None),
                lambda: lib.dh_relu(None, buf.ptr, 8, None),
                lambda: lib.dh_add(src.ptr, None, buf.ptr, 8, None),
                lambda: lib.dh_bias_add(src.ptr, None, buf.ptr, 2, 4, None),
                lambda: lib.dh_gemm_nn(src.ptr, None, None, buf.ptr, 2, 2, 2, None),
                lambda: lib.dh_adam_step(buf.ptr, buf.ptr, None, src.ptr, 0.5, 0.5, 0.9, 0.1, 0.1, 1e-8, 8, None)):
        with pytest.raises(A.HipError):
            A.check(bad())


@pytest.mark.parametrize("rows,cols", [(4096, 64), (65536, 3), (1024, 512), (16384, 128), (7, 5), (64, 8192)])
def test_bias_gradient_in_parts_through_adam(be, orc, rows, cols):
    """dh_bias_grad_parts / dh_act_bias_grad_parts leave the column sums as row-range sums;
    dh_adam_step_multi fed with them gives, to the bit, what it gives when fed with dh_bias_grad's
    result -- with one gradient, with two, and with one of the two in plain form."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    rng = np.random.default_rng(rows + cols)
    z = rng.uniform(-2, 2, (rows, cols)).astype(np.float32)
    d1 = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    d2 = rng.uniform(-1, 1, (rows, cols)).astype(np.float32)
    parts1 = be.bias_grad_parts(d1)
    assert parts1.shape == (be.lib.dh_bias_grad_part_count(rows, cols), cols)
    plain1 = be.bias_grad(d1)
    close(parts1.astype(np.float64).sum(axis=0).astype(np.float32), orc.bias_grad(d1), scale=max(1.0, np.sqrt(rows)))
    dz_ref, plain2 = be.act_bias_grad(z, d2, A.ACT_LEAKY, 0.2)
    dz, parts2 = be.act_bias_grad_parts(z, d2, A.ACT_LEAKY, 0.2)
    np.testing.assert_array_equal(dz, dz_ref)
    p = rng.standard_normal(cols).astype(np.float32)
    m = (rng.standard_normal(cols) * 0.1).astype(np.float32)
    v = (rng.uniform(0, 1, cols) * 0.01).astype(np.float32)
    lrt = 1e-3
    want = be.adam_step_multi([(p, m, v, plain1, None, lrt), (p, m, v, plain1, plain2, lrt), (p, m, v, plain2, plain1, lrt)],
                              0.5, 0.999, 1e-8)
    got = be.adam_step_multi([(p, m, v, parts1, None, lrt), (p, m, v, parts1, parts2, lrt), (p, m, v, plain2, parts1, lrt)],
                             0.5, 0.999, 1e-8)
    for w, g in zip(want, got):
        for a, b in zip(w, g):
            np.testing.assert_array_equal(a, b)


def test_column_sums_of_unaligned_tensors(be, orc):
    """Column counts divisible by 4 take the kernel whose lanes own 4 adjacent columns; tensors that
    do not start on a 16-byte boundary go through its element-wise accesses."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    rng = np.random.default_rng(9)
    rows, cols = 777, 36
    z = rng.uniform(-2, 2, rows * cols + 1).astype(np.float32)
    d = rng.uniform(-1, 1, rows * cols + 1).astype(np.float32)
    dz_buf, db = A.Buf(rows * cols + 1), A.Buf(cols)
    zb, dbuf = A.Buf.from_numpy(z), A.Buf.from_numpy(d)
    A.check(be.lib.dh_act_bias_grad(zb.ptr + 4, dbuf.ptr + 4, dz_buf.ptr + 4, db.ptr, rows, cols, A.ACT_LEAKY, 0.2, None))
    z2, d2 = z[1:].reshape(rows, cols), d[1:].reshape(rows, cols)
    exp = orc.leaky_relu_grad(z2, d2, 0.2)
    np.testing.assert_array_equal(dz_buf.numpy()[1:].reshape(rows, cols), exp)
    close(db.numpy(), orc.bias_grad(exp), scale=np.sqrt(rows))
    A.check(be.lib.dh_bias_grad(dbuf.ptr + 4, db.ptr, rows, cols, None))
    close(db.numpy(), orc.bias_grad(d2), scale=np.sqrt(rows))


def test_staged_host_to_device_copies(be):
    """dh_memcpy_h2d_staged: the host buffer may be overwritten as soon as the call returns, copies are
    ordered with the kernels of their stream, and more copies than there are staging buffers (16), of
    growing and shrinking sizes, all arrive intact."""
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = be.lib
    rng = np.random.default_rng(11)
    sizes = [1, 100, 786432, 6400, 3, 70000, 2, 1 << 20] * 5          # 40 copies
    host = np.empty(max(sizes), np.float32)
    bufs, expected = [], []
    for n in sizes:
        vals = rng.standard_normal(n).astype(np.float32)
        host[:n] = vals                                              # the one host buffer, reused every time
        d = A.Buf((n,))
        A.check(lib.dh_memcpy_h2d_staged(d.ptr, host.ctypes.data, n * 4, None))
        host[:n] = -1.0
        out = A.Buf((n,))
        A.check(lib.dh_relu(d.ptr, out.ptr, n, None))                # queued behind the copy on the same stream
        bufs.append((d, out))
        expected.append(vals)
    for (d, out), vals in zip(bufs, expected):
        np.testing.assert_array_equal(d.numpy(), vals)
        np.testing.assert_array_equal(out.numpy(), np.maximum(vals, 0.0))
    # nothing to copy / null pointers
    A.check(lib.dh_memcpy_h2d_staged(bufs[0][0].ptr, host.ctypes.data, 0, None))
    assert lib.dh_memcpy_h2d_staged(None, host.ctypes.data, 4, None) != 0

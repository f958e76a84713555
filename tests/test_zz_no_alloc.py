"""dh_bias_grad_static -- the column sums for callers that cannot allocate -- against dh_bias_grad
through the C ABI: bit-identical results on two calls in a row, the second on a smaller matrix (the
fixed scratch buffer keeps the first call's range sums), no growth of the library's arenas, and a clear
refusal of a matrix whose range sums do not fit the buffer."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def both(A, lib, dz):
    rows, cols = dz.shape
    d = A.Buf.from_numpy(dz)
    ref, got = A.Buf((cols,)), A.Buf((cols,))
    A.check(lib.dh_memset0(got.ptr, cols * 4, None))
    A.check(lib.dh_bias_grad(d.ptr, ref.ptr, rows, cols, None))
    before, pool = lib.dh_workspace_bytes(), A.pool_stats()
    A.check(lib.dh_bias_grad_static(d.ptr, got.ptr, rows, cols, None))
    assert lib.dh_workspace_bytes() == before
    assert A.pool_stats() == pool           # no hipMalloc, no block handed out by the tensor pool either
    return ref.numpy(), got.numpy()


def test_static_bias_gradient_equals_the_allocating_one(orc):
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    rng = np.random.default_rng(3)
    # [64*16*16, 128]: 1024 row ranges of 128 columns, then a smaller and narrower matrix whose range
    # sums overwrite only the head of the buffer, then 3 columns (the scalar kernel) and one range
    for shape in ((16384, 128), (1000, 36), (4099, 3), (3, 8)):
        print("shape", shape, flush=True)
        dz = rng.uniform(-1, 1, shape).astype(np.float32)
        ref, got = both(A, lib, dz)
        np.testing.assert_array_equal(got, ref)
        exp = orc.bias_grad(dz)
        np.testing.assert_allclose(got, exp, rtol=1e-4, atol=1e-5 * max(1.0, float(np.abs(exp).max())))


def test_static_bias_gradient_refuses_what_does_not_fit():
    import __graft_entry__ as ge
    A = ge.load_package().hipabi
    lib = A.load()
    rows, cols = 8192, 1024
    need = lib.dh_bias_grad_part_count(rows, cols) * cols * 4
    assert need > lib.dh_bias_grad_static_max_bytes()
    d, out = A.Buf((rows, cols)), A.Buf((cols,))
    with pytest.raises(A.HipError, match="fixed buffer"):
        A.check(lib.dh_bias_grad_static(d.ptr, out.ptr, rows, cols, None))

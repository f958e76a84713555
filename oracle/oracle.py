"""ctypes front-end of the CPU oracle -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Loads ``oracle/liboracle.so`` (the C restatement, ``orc_*`` / ``orc_*_f64``) and, when it was
built, ``oracle/_ref/libdcgan_ref.so`` (the reference's own CPU operators, ``ref_*``), and
exposes one numpy-level function per operator.  ``Oracle("orc")`` is the fp32 restatement,
``Oracle("orc", f64=True)`` its float64-accumulating twin and ``Oracle("ref")`` the reference
build; all three take the same arguments.

Only tests, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` import this.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_ORACLE = os.path.join(HERE, "liboracle.so")
LIB_REF = os.path.join(HERE, "_ref", "libdcgan_ref.so")

_fp = C.POINTER(C.c_float)


def build(verbose=False):
    """Compile liboracle.so (and _ref when the reference tree is mounted)."""
    out = subprocess.run(["make", "-C", HERE, "all"], capture_output=True, text=True)
    if out.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + out.stdout + out.stderr)
    if verbose:
        print(out.stdout)


def have_ref():
    return os.path.exists(LIB_REF)


def same_pad(n_in, k, s):
    """(pad_total, out) of the reference's SAME rule (src/ops/conv2d.cu:26-46)."""
    p = k - s if n_in % s == 0 else k - (n_in % s)
    return max(p, 0), -(-n_in // s)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(_fp)


class Oracle:
    def __init__(self, flavour="orc", f64=False):
        assert flavour in ("orc", "ref")
        path = LIB_ORACLE if flavour == "orc" else LIB_REF
        if not os.path.exists(path):
            raise FileNotFoundError(path + " is not built (run `make -C oracle`)")
        self.lib = C.CDLL(path)
        self.prefix = flavour + "_"
        self.suffix = "_f64" if (f64 and flavour == "orc") else ""
        self.flavour = flavour

    def _fn(self, name, restype=None):
        f = getattr(self.lib, self.prefix + name + self.suffix)
        f.restype = restype
        return f

    def set_threads(self, n):
        if self.flavour == "orc":
            self._fn("set_threads")(C.c_int(n))

    # ---- convolutions -------------------------------------------------------------------
    def conv2d(self, x, k, strides=(2, 2), pads=None):
        x, k = _f32(x), _f32(k)
        N, H, W, Cc = x.shape
        kh, kw, C2, O = k.shape
        assert C2 == Cc
        if pads is None:
            pads = (same_pad(H, kh, strides[0])[0], same_pad(W, kw, strides[1])[0])
        Ho, Wo = -(-H // strides[0]), -(-W // strides[1])
        y = np.empty((N, Ho, Wo, O), np.float32)
        self._fn("conv2d")(_p(x), _p(k), _p(y), *map(C.c_int, (N, H, W, Cc, kh, kw, O,
                           strides[0], strides[1], pads[0], pads[1])))
        return y

    def conv2d_input_grad(self, dy, k, stride, in_hw):
        dy, k = _f32(dy), _f32(k)
        N, Ho, Wo, O = dy.shape
        kh, kw, Cc, O2 = k.shape
        assert O2 == O
        dx = np.zeros((N, in_hw[0], in_hw[1], Cc), np.float32)
        self._fn("conv2d_input_grad")(_p(dy), _p(k), _p(dx), *map(C.c_int, (
            N, Ho, Wo, O, kh, kw, Cc, stride, in_hw[0], in_hw[1])))
        return dx

    def conv2d_kernel_grad(self, dy, x, stride, pads, k_hw=None):
        dy, x = _f32(dy), _f32(x)
        N, Ho, Wo, O = dy.shape
        N2, H, W, Cc = x.shape
        assert N2 == N
        kh = H + pads[0] - stride * (Ho - 1)
        kw = W + pads[1] - stride * (Wo - 1)
        if k_hw is not None:
            assert (kh, kw) == tuple(k_hw)
        dk = np.zeros((kh, kw, Cc, O), np.float32)
        self._fn("conv2d_kernel_grad")(_p(dy), _p(x), _p(dk), *map(C.c_int, (
            N, Ho, Wo, O, H, W, Cc, stride, pads[0], pads[1])))
        return dk

    def conv2d_transpose(self, x, k, out_hw, stride):
        x, k = _f32(x), _f32(k)
        N, Hi, Wi, Ci = x.shape
        kh, kw, Co, Ci2 = k.shape
        assert Ci2 == Ci
        y = np.zeros((N, out_hw[0], out_hw[1], Co), np.float32)
        self._fn("conv2d_transpose")(_p(x), _p(k), _p(y), *map(C.c_int, (
            N, Hi, Wi, Ci, kh, kw, Co, stride, out_hw[0], out_hw[1])))
        return y

    def conv2d_transpose_input_grad(self, dy, k, stride, in_hw):
        dy, k = _f32(dy), _f32(k)
        N, Hy, Wy, Co = dy.shape
        kh, kw, Co2, Ci = k.shape
        assert Co2 == Co
        dx = np.zeros((N, in_hw[0], in_hw[1], Ci), np.float32)
        self._fn("conv2d_transpose_input_grad")(_p(dy), _p(k), _p(dx), *map(C.c_int, (
            N, Hy, Wy, Co, kh, kw, Ci, stride, in_hw[0], in_hw[1])))
        return dx

    def conv2d_transpose_kernel_grad(self, dy, x, stride, k_hw):
        dy, x = _f32(dy), _f32(x)
        N, Hy, Wy, Co = dy.shape
        N2, Hi, Wi, Ci = x.shape
        assert N2 == N
        dk = np.zeros((k_hw[0], k_hw[1], Co, Ci), np.float32)
        self._fn("conv2d_transpose_kernel_grad")(_p(dy), _p(x), _p(dk), *map(C.c_int, (
            N, Hy, Wy, Co, Hi, Wi, Ci, stride, k_hw[0], k_hw[1])))
        return dk

    # ---- bias, activations --------------------------------------------------------------
    def bias_add(self, z, b):
        z, b = _f32(z), _f32(b)
        out = np.empty_like(z)
        cols = z.shape[-1]
        self._fn("mvrow_add")(_p(z), _p(b), _p(out), C.c_size_t(z.size // cols), C.c_size_t(cols))
        return out

    def bias_grad(self, dz):
        dz = _f32(dz)
        cols = dz.shape[-1]
        out = np.empty((cols,), np.float32)
        self._fn("mat_sum_cols")(_p(dz), _p(out), C.c_size_t(dz.size // cols), C.c_size_t(cols))
        return out

    def mat_sum_rows(self, a):
        a = _f32(a)
        out = np.empty((a.shape[0],), np.float32)
        self._fn("mat_sum_rows")(_p(a), _p(out), C.c_size_t(a.shape[0]), C.c_size_t(a.shape[1]))
        return out

    def _unary(self, name, a, *extra):
        a = _f32(a)
        out = np.empty_like(a)
        self._fn(name)(_p(a), _p(out), C.c_size_t(a.size), *extra)
        return out

    def _binary(self, name, a, b, *extra_before_n):
        a, b = _f32(a), _f32(b)
        assert a.shape == b.shape
        out = np.empty_like(a)
        self._fn(name)(_p(a), _p(b), _p(out), *extra_before_n, C.c_size_t(a.size))
        return out

    def relu(self, a):
        return self._unary("relu", a)

    def relu_leaky(self, a, alpha=0.2):
        return self._unary("relu_leaky", a, C.c_float(alpha))

    def tanh(self, a):
        return self._unary("tanh", a)

    def sigmoid(self, a):
        return self._unary("sigmoid", a)

    def relu_grad(self, z, dout):
        return self._binary("relu_grad", z, dout)

    def leaky_relu_grad(self, z, dout, alpha):
        return self._binary("leaky_relu_grad", z, dout, C.c_float(alpha))

    def tanh_grad(self, t, dout):
        return self._binary("tanh_grad", t, dout)

    def sigmoid_grad(self, s, dout):
        return self._binary("sigmoid_grad", s, dout)

    def add(self, a, b):
        return self._binary("add", a, b)

    # ---- losses -------------------------------------------------------------------------
    def sigmoid_cross_entropy(self, y, logits):
        y, logits = _f32(y), _f32(logits)
        return np.float32(self._fn("sigmoid_cross_entropy", C.c_float)(
            _p(y), _p(logits), C.c_size_t(y.size)))

    def sigmoid_cross_entropy_grad(self, y, logits):
        return self._binary("sigmoid_cross_entropy_grad", y, logits)

    def mse(self, y, y_hat):
        y, y_hat = _f32(y), _f32(y_hat)
        return np.float32(self._fn("mse", C.c_float)(_p(y), _p(y_hat), C.c_size_t(y.shape[0]),
                                                     C.c_size_t(y.size // y.shape[0])))

    def mse_grad(self, y, y_hat):
        return self._binary("mse_grad", y, y_hat)

    def argmax_acc(self, y, y_hat):
        y, y_hat = _f32(y), _f32(y_hat)
        return int(self._fn("argmax_acc", C.c_size_t)(_p(y), _p(y_hat), C.c_size_t(y.shape[0]),
                                                      C.c_size_t(y.shape[1])))

    # ---- dense --------------------------------------------------------------------------
    def _mm(self, name, a, b, m, n, p):
        a, b = _f32(a), _f32(b)
        out = np.empty((m, p), np.float32)
        self._fn(name)(_p(a), _p(b), _p(out), C.c_size_t(m), C.c_size_t(n), C.c_size_t(p))
        return out

    def mm_mul(self, a, b):          # (m,n) x (n,p)
        return self._mm("mm_mul", a, b, a.shape[0], a.shape[1], b.shape[1])

    def tmm_mul(self, a, b):         # tr(a) x b, a (n,m), b (n,p)
        return self._mm("tmm_mul", a, b, a.shape[1], a.shape[0], b.shape[1])

    def mtm_mul(self, a, b):         # a x tr(b), a (m,n), b (p,n)
        return self._mm("mtm_mul", a, b, a.shape[0], a.shape[1], b.shape[0])

    def mat_mul_add(self, x, w, b):
        x, w, b = _f32(x), _f32(w), _f32(b)
        out = np.empty((x.shape[0], w.shape[1]), np.float32)
        self._fn("mat_mul_add")(_p(x), _p(w), _p(b), _p(out), C.c_size_t(x.shape[0]),
                                C.c_size_t(x.shape[1]), C.c_size_t(w.shape[1]))
        return out

    # ---- Adam ---------------------------------------------------------------------------
    def moment_update(self, var, dv, a, b):
        var, dv = _f32(var).copy(), _f32(dv)
        self._fn("moment_update")(_p(dv), _p(var), C.c_float(a), C.c_float(b), C.c_size_t(var.size))
        return var

    def moment_update2(self, var, dv, a, b):
        var, dv = _f32(var).copy(), _f32(dv)
        self._fn("moment_update2")(_p(dv), _p(var), C.c_float(a), C.c_float(b), C.c_size_t(var.size))
        return var

    @staticmethod
    def adam_lrt(t, lr, beta1, beta2):
        """Host-side step size of src/cpu/kernels.cu:193-206 in float arithmetic.
        Returns (t + 1, lrt)."""
        f = np.float32
        t = f(f(t) + f(1))
        lrt = f(lr) * np.sqrt(f(1) - np.power(f(beta2), t, dtype=f), dtype=f) \
            / (f(1) - np.power(f(beta1), t, dtype=f))
        return t, f(lrt)

    def adam_apply(self, p, m, v, lrt, eps):
        p, m, v = _f32(p).copy(), _f32(m), _f32(v)
        self._fn("adam_apply")(_p(m), _p(v), _p(p), C.c_float(lrt), C.c_float(eps),
                               C.c_size_t(p.size))
        return p

    def vect_update(self, var, dv, coeff):
        var, dv = _f32(var).copy(), _f32(dv)
        self._fn("vect_update")(_p(dv), _p(var), C.c_float(coeff), C.c_size_t(var.size))
        return var


class XorShift:
    """The reference's seeded generator (src/utils/xorshift.cu:13-40): floats in [0, 1]."""

    class _State(C.Structure):
        _fields_ = [("s", C.c_uint64 * 4)]

    def __init__(self, seed):
        self.lib = C.CDLL(LIB_ORACLE)
        self.state = self._State()
        self.lib.orc_xorshift_seed(C.byref(self.state), C.c_uint64(seed))

    def f32(self, shape):
        out = np.empty(shape, np.float32)
        self.lib.orc_xorshift_fill(C.byref(self.state), _p(out), C.c_size_t(out.size))
        return out

    def next_u64(self):
        self.lib.orc_xorshift_next_u64.restype = C.c_uint64
        return int(self.lib.orc_xorshift_next_u64(C.byref(self.state)))


class RefProgram:
    """A node list run by the reference's own runtime (oracle/_ref only): sequentially, as under
    RT_MODE=CPU (src/cpu/runner.cu:10-14), or by rt::optimize + cpu::ThreadPoolRunner, as under
    RT_MODE=MCPU (src/ops/graph.cu:180-192; the reference hard-codes 4 workers, :32).  The
    reference's optimiser does not split convolution nodes (src/runtime/optimizer.cu:239-247,
    :561-583), so MCPU runs each convolution on one worker and gains only from nodes that are
    independent of each other."""

    def __init__(self):
        if not have_ref():
            raise FileNotFoundError(LIB_REF + " is not built (needs the reference tree)")
        self.lib = C.CDLL(LIB_REF)
        self.lib.ref_program_new.restype = C.c_void_p
        self.p = C.c_void_p(self.lib.ref_program_new())
        self.keep = []          # operand arrays stay alive as long as the program
        self.count = 0

    def __del__(self):
        if getattr(self, "p", None):
            self.lib.ref_program_free(self.p)
            self.p = None

    @staticmethod
    def _ints(v):
        return (C.c_int * len(v))(*v)

    def _preds(self, preds):
        return self._ints(list(preds) or [-1]), C.c_int(len(preds))

    def _added(self, idx):
        self.count += 1
        assert idx == self.count - 1
        return idx

    def conv2d(self, x, k, strides, pads, preds=()):
        x, k = _f32(x), _f32(k)
        N, H, W, _ = x.shape
        y = np.zeros((N, -(-H // strides[0]), -(-W // strides[1]), k.shape[3]), np.float32)
        self.keep += [x, k, y]
        pa, pn = self._preds(preds)
        idx = self.lib.ref_node_conv2d(self.p, _p(x), _p(k), _p(y), self._ints(strides),
                                       C.c_int(pads[0]), C.c_int(pads[1]),
                                       self._ints(x.shape), self._ints(k.shape), pa, pn)
        return self._added(idx), y

    def conv2d_input_grad(self, dy, k, stride, in_hw, preds=()):
        dy, k = _f32(dy), _f32(k)
        dx = np.zeros((dy.shape[0], in_hw[0], in_hw[1], k.shape[2]), np.float32)
        self.keep += [dy, k, dx]
        pa, pn = self._preds(preds)
        idx = self.lib.ref_node_conv2d_input_grad(self.p, _p(dy), _p(k), _p(dx),
                                                  self._ints((stride, stride)), self._ints(dy.shape),
                                                  self._ints(k.shape), self._ints(dx.shape), pa, pn)
        return self._added(idx), dx

    def conv2d_kernel_grad(self, dy, x, stride, pads, preds=()):
        dy, x = _f32(dy), _f32(x)
        kh = x.shape[1] + pads[0] - stride * (dy.shape[1] - 1)
        kw = x.shape[2] + pads[1] - stride * (dy.shape[2] - 1)
        dk = np.zeros((kh, kw, x.shape[3], dy.shape[3]), np.float32)
        self.keep += [dy, x, dk]
        pa, pn = self._preds(preds)
        idx = self.lib.ref_node_conv2d_kernel_grad(self.p, _p(dy), _p(x), _p(dk),
                                                   self._ints((stride, stride)), self._ints(dy.shape),
                                                   self._ints(x.shape), self._ints(pads), pa, pn)
        return self._added(idx), dk

    def run(self, outs, mcpu=False, workers=4):
        self.lib.ref_program_run(self.p, self._ints(outs), C.c_int(len(outs)),
                                 C.c_int(1 if mcpu else 0), C.c_int(workers))

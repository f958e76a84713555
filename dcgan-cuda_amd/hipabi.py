"""ctypes binding of the C ABI (include/dcgan_hip.h) plus a numpy-level front-end.

`load()` returns the CDLL with every entry point typed; it raises if the library has not been
built -- there is no CPU fallback.  `HipBackend` offers one method per operator with numpy arrays
in and out (host<->device copies through dh_memcpy_*), under the same names as the CPU oracle's
front-end so that parity tests can drive either.  `Buf` is a device allocation for callers that
keep data resident (the benchmark does).
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
# DCGAN_HIP_LIB overrides the library file (A/B runs of an experimental build)
LIB_PATH = os.environ.get("DCGAN_HIP_LIB") or os.path.join(HERE, "lib", "libdcgan_hip.so")

ACT_NONE, ACT_RELU, ACT_LEAKY, ACT_TANH, ACT_SIGMOID = range(5)

_vp, _sz, _i, _f = C.c_void_p, C.c_size_t, C.c_int, C.c_float

# name -> argtypes (every function returns int unless listed in _RESTYPES)
_SIGS = {
    "dh_init": [_i],
    "dh_device_info": [C.c_char_p, _sz, C.POINTER(_i), C.POINTER(_i), C.POINTER(_sz)],
    "dh_malloc": [C.POINTER(_vp), _sz],
    "dh_free": [_vp],
    "dh_memcpy_h2d": [_vp, _vp, _sz],
    "dh_memcpy_h2d_staged": [_vp, _vp, _sz, _vp],
    "dh_memcpy_d2h": [_vp, _vp, _sz],
    "dh_memcpy_d2d": [_vp, _vp, _sz, _vp],
    "dh_memset0": [_vp, _sz, _vp],
    "dh_sync": [],
    "dh_stream_create": [C.POINTER(_vp)],
    "dh_stream_wait_event": [_vp, _vp],
    "dh_stream_destroy": [_vp],
    "dh_stream_sync": [_vp],
    "dh_event_create": [C.POINTER(_vp)],
    "dh_event_destroy": [_vp],
    "dh_event_record": [_vp, _vp],
    "dh_event_elapsed_ms": [_vp, _vp, C.POINTER(_f)],
    "dh_workspace_reserve": [_sz],
    "dh_pool_alloc": [C.POINTER(_vp), _sz],
    "dh_pool_free": [_vp],
    "dh_pool_reserve": [_sz],
    "dh_pool_trim": [],
    "dh_pool_stats": [C.POINTER(_sz)] * 4,
    "dh_debug_force_generic_conv": [_i],
    "dh_debug_force_splitk": [_i],
    "dh_debug_force_tile_width": [_i],
    "dh_sigmoid_cross_entropy_head": [_vp] * 9 + [_sz, _vp],
    "dh_gemm_nn_act": [_vp] * 4 + [_sz] * 3 + [_i, _f, _vp],
    "dh_gemm_tn_pair": [_vp] * 5 + [_sz] * 3 + [_vp],
    "dh_gemm_tn_pair_supported": [_sz] * 3,
    "dh_profile_enable": [_i],
    "dh_profile_reset": [],
    "dh_profile_read": [C.c_char_p, _sz],
    "dh_conv2d_fwd": [_vp, _vp, _vp] + [_i] * 13 + [_vp, _i, _f, _vp],
    "dh_conv2d_dx": [_vp, _vp, _vp] + [_i] * 13 + [_vp, _i, _f, _vp],
    "dh_conv2d_dk": [_vp, _vp, _vp] + [_i] * 13 + [_vp],
    "dh_conv2d_fwd_pair": [_vp] * 5 + [_i] * 13 + [_vp, _i, _f, _vp],
    "dh_conv2d_dx_pair": [_vp] * 5 + [_i] * 13 + [_vp, _i, _f, _vp],
    "dh_conv2d_dk_pair": [_vp] * 5 + [_i] * 13 + [_vp],
    "dh_conv2d_dk_pair_supported": [_i] * 11,
    "dh_conv2d_fwd_pair_supported": [_i] * 13,
    "dh_bias_add": [_vp, _vp, _vp, _sz, _sz, _vp],
    "dh_bias_grad": [_vp, _vp, _sz, _sz, _vp],
    "dh_bias_grad_parts": [_vp, _vp, _sz, _sz, _vp],
    "dh_bias_grad_static": [_vp, _vp, _sz, _sz, _vp],
    "dh_mat_sum_rows": [_vp, _vp, _sz, _sz, _vp],
    "dh_relu": [_vp, _vp, _sz, _vp],
    "dh_relu_leaky": [_vp, _vp, _sz, _f, _vp],
    "dh_tanh": [_vp, _vp, _sz, _vp],
    "dh_sigmoid": [_vp, _vp, _sz, _vp],
    "dh_relu_grad": [_vp, _vp, _vp, _sz, _vp],
    "dh_leaky_relu_grad": [_vp, _vp, _vp, _f, _sz, _vp],
    "dh_tanh_grad": [_vp, _vp, _vp, _sz, _vp],
    "dh_sigmoid_grad": [_vp, _vp, _vp, _sz, _vp],
    "dh_add": [_vp, _vp, _vp, _sz, _vp],
    "dh_act_bias_grad": [_vp, _vp, _vp, _vp, _sz, _sz, _i, _f, _vp],
    "dh_act_bias_grad_parts": [_vp, _vp, _vp, _vp, _sz, _sz, _i, _f, _vp],
    "dh_sigmoid_cross_entropy": [_vp, _vp, _vp, _sz, _vp],
    "dh_sigmoid_cross_entropy_grad": [_vp, _vp, _vp, _sz, _vp],
    "dh_mse": [_vp, _vp, _vp, _sz, _sz, _vp],
    "dh_mse_grad": [_vp, _vp, _vp, _sz, _vp],
    "dh_argmax_acc": [_vp, _vp, _vp, _sz, _sz, _vp],
    "dh_gemm_nn": [_vp, _vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "dh_gemm_tn": [_vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "dh_gemm_nt": [_vp, _vp, _vp, _sz, _sz, _sz, _vp],
    "dh_moment_update": [_vp, _vp, _f, _f, _sz, _vp],
    "dh_moment_update2": [_vp, _vp, _f, _f, _sz, _vp],
    "dh_adam_update": [_vp, _vp, _vp, _f, _f, _sz, _vp],
    "dh_adam_step": [_vp, _vp, _vp, _vp, _f, _f, _f, _f, _f, _f, _sz, _vp],
    "dh_adam_step_multi": [_vp, _i, _f, _f, _f, _f, _f, _vp],
    "dh_sgd_update": [_vp, _vp, _vp, _sz, _vp],
}
# name -> result type, or (result type, argtypes)
_RESTYPES = {"dh_version": C.c_char_p, "dh_last_error": C.c_char_p, "dh_workspace_bytes": _sz,
             "dh_bias_grad_static_max_bytes": _sz,
             "dh_bias_grad_part_count": (_sz, [_sz, _sz])}

_lib = None


def load():
    """The typed CDLL.  Raises RuntimeError when lib/libdcgan_hip.so is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is not built; run `python dcgan-cuda_amd/build.py` "
                               "(there is no CPU fallback)" % LIB_PATH)
        lib = C.CDLL(LIB_PATH)
        for name, args in _SIGS.items():
            fn = getattr(lib, name)
            fn.argtypes = args
            fn.restype = _i
        for name, res in _RESTYPES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res if isinstance(res, tuple) else (res, [])
        _lib = lib
    return _lib


def exported_symbols():
    return sorted(list(_SIGS) + list(_RESTYPES))


class HipError(RuntimeError):
    pass


def check(rc):
    if rc != 0:
        raise HipError("dcgan_hip error %d: %s" % (rc, load().dh_last_error().decode()))


class Buf:
    """A device allocation of fp32 elements."""

    def __init__(self, shape):
        self.shape = tuple(int(s) for s in (shape if hasattr(shape, "__len__") else (shape,)))
        self.size = int(np.prod(self.shape)) if self.shape else 1
        p = _vp()
        check(load().dh_malloc(C.byref(p), self.size * 4))
        self.ptr = p.value

    @classmethod
    def from_numpy(cls, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        b = cls(a.shape)
        b.write(a)
        return b

    @classmethod
    def zeros(cls, shape):
        b = cls(shape)
        check(load().dh_memset0(b.ptr, b.size * 4, None))
        return b

    def write(self, a):
        a = np.ascontiguousarray(a, dtype=np.float32)
        assert a.size == self.size
        check(load().dh_memcpy_h2d(self.ptr, a.ctypes.data, a.size * 4))

    def numpy(self):
        out = np.empty(self.shape, np.float32)
        check(load().dh_memcpy_d2h(out.ctypes.data, self.ptr, self.size * 4))
        return out

    def free(self):
        if self.ptr:
            check(load().dh_free(self.ptr))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def pool_stats():
    """hipMalloc calls, bytes held, bytes handed out and their peak of the tensor pool (dh_pool_*)."""
    v = [_sz() for _ in range(4)]
    check(load().dh_pool_stats(*[C.byref(x) for x in v]))
    return dict(zip(("hipmallocs", "held", "in_use", "peak"), (x.value for x in v)))


def device_info():
    name = C.create_string_buffer(256)
    cus, khz, mem = _i(), _i(), _sz()
    check(load().dh_device_info(name, 256, C.byref(cus), C.byref(khz), C.byref(mem)))
    return {"name": name.value.decode(), "compute_units": cus.value, "clock_khz": khz.value,
            "memory_bytes": mem.value}


class AdamItem(C.Structure):
    """dh_adam_item of include/dcgan_hip.h."""
    _fields_ = [("p", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p), ("g1", C.c_void_p), ("g2", C.c_void_p),
                ("n", C.c_size_t), ("lrt", C.c_float), ("g1_parts", C.c_size_t), ("g2_parts", C.c_size_t)]


class Timer:
    """HIP-event timer on a given stream (None = the default stream)."""

    def __init__(self, stream=None):
        self.stream = stream
        self.e0, self.e1 = _vp(), _vp()
        check(load().dh_event_create(C.byref(self.e0)))
        check(load().dh_event_create(C.byref(self.e1)))

    def start(self):
        check(load().dh_event_record(self.e0, self.stream))

    def stop_ms(self):
        check(load().dh_event_record(self.e1, self.stream))
        ms = _f()
        check(load().dh_event_elapsed_ms(self.e0, self.e1, C.byref(ms)))
        return ms.value


def profile_enable(on):
    """0/False off, 1/True the convolution kernels, 2 every tagged kernel."""
    check(load().dh_profile_enable(int(on)))


def profile_reset():
    check(load().dh_profile_reset())


def profile_read():
    """[{name, launches, ms, flops, issued}] per kernel tag since the last reset.  `flops` is the
    algorithmic work of the launches: FLOPs, or bytes for the tags that start with "hbm:"; `issued` the
    FLOPs the matrix cores were issued (0.0 where the launch site does not account for them)."""
    buf = C.create_string_buffer(1 << 16)
    check(load().dh_profile_read(buf, len(buf)))
    rows = []
    for line in buf.value.decode().splitlines():
        name, n, ms, fl, issued = line.split("\t")
        rows.append({"name": name, "launches": int(n), "ms": float(ms), "flops": float(fl), "issued": float(issued)})
    return rows


def same_pad(n_in, k, s):
    """(pad_total, out) of the reference's SAME rule (src/ops/conv2d.cu:26-46)."""
    p = k - s if n_in % s == 0 else k - (n_in % s)
    return max(p, 0), -(-n_in // s)


class HipBackend:
    """numpy in, numpy out; every call runs the HIP kernels through the C ABI and copies back."""

    def __init__(self, device=0, stream=None):
        self.lib = load()
        check(self.lib.dh_init(device))
        self.stream = stream

    # -- helpers --
    def _up(self, *arrays):
        return [Buf.from_numpy(a) for a in arrays]

    # -- convolutions --
    def conv2d(self, x, k, strides=(2, 2), pads=None, bias=None, act=ACT_NONE, alpha=0.0):
        N, H, W, Cc = x.shape
        kh, kw, C2, O = k.shape
        assert C2 == Cc
        if pads is None:
            pads = (same_pad(H, kh, strides[0])[0], same_pad(W, kw, strides[1])[0])
        Ho, Wo = -(-H // strides[0]), -(-W // strides[1])
        dx, dk = self._up(x, k)
        db = Buf.from_numpy(bias) if bias is not None else None
        y = Buf((N, Ho, Wo, O))
        check(self.lib.dh_conv2d_fwd(dx.ptr, dk.ptr, y.ptr, N, H, W, Cc, kh, kw, O, strides[0], strides[1],
                                     pads[0] // 2, pads[1] // 2, Ho, Wo, db.ptr if db else None, act, alpha,
                                     self.stream))
        return y.numpy()

    def conv2d_pair(self, x1, x2, k, strides=(2, 2), bias=None, act=ACT_NONE, alpha=0.0):
        """conv2d of two inputs of one shape with the same filter, in one launch -> (y1, y2)."""
        N, H, W, Cc = x1.shape
        assert x2.shape == x1.shape
        kh, kw, C2, O = k.shape
        pads = (same_pad(H, kh, strides[0])[0], same_pad(W, kw, strides[1])[0])
        Ho, Wo = -(-H // strides[0]), -(-W // strides[1])
        d1, d2, dk = self._up(x1, x2, k)
        db = Buf.from_numpy(bias) if bias is not None else None
        y1, y2 = Buf((N, Ho, Wo, O)), Buf((N, Ho, Wo, O))
        check(self.lib.dh_conv2d_fwd_pair(d1.ptr, d2.ptr, dk.ptr, y1.ptr, y2.ptr, N, H, W, Cc, kh, kw, O, strides[0],
                                          strides[1], pads[0] // 2, pads[1] // 2, Ho, Wo, db.ptr if db else None, act,
                                          alpha, self.stream))
        return y1.numpy(), y2.numpy()

    def conv2d_input_grad_pair(self, dy1, dy2, k, stride, in_hw, bias=None, act=ACT_NONE, alpha=0.0):
        """conv2d_input_grad of two gradients of one shape with the same filter, in one launch."""
        N, Ho, Wo, O = dy1.shape
        assert dy2.shape == dy1.shape
        kh, kw, Cc, O2 = k.shape
        H, W = in_hw
        pad_h = (Ho - 1) * stride + kh - H
        pad_w = (Wo - 1) * stride + kw - W
        d1, d2, dk = self._up(dy1, dy2, k)
        db = Buf.from_numpy(bias) if bias is not None else None
        o1, o2 = Buf((N, H, W, Cc)), Buf((N, H, W, Cc))
        check(self.lib.dh_conv2d_dx_pair(d1.ptr, d2.ptr, dk.ptr, o1.ptr, o2.ptr, N, Ho, Wo, O, kh, kw, Cc, stride,
                                         stride, pad_h // 2, pad_w // 2, H, W, db.ptr if db else None, act, alpha,
                                         self.stream))
        return o1.numpy(), o2.numpy()

    def conv2d_kernel_grad_pair(self, dy1, x1, dy2, x2, stride, pads):
        """conv2d_kernel_grad(dy1, x1) + conv2d_kernel_grad(dy2, x2) as one contraction."""
        N, Ho, Wo, O = dy1.shape
        _, H, W, Cc = x1.shape
        kh = H + pads[0] - stride * (Ho - 1)
        kw = W + pads[1] - stride * (Wo - 1)
        a1, b1, a2, b2 = self._up(x1, dy1, x2, dy2)
        out = Buf((kh, kw, Cc, O))
        check(self.lib.dh_conv2d_dk_pair(a1.ptr, b1.ptr, a2.ptr, b2.ptr, out.ptr, N, H, W, Cc, Ho, Wo, O, kh, kw,
                                         stride, stride, pads[0] // 2, pads[1] // 2, self.stream))
        return out.numpy()

    def conv2d_input_grad(self, dy, k, stride, in_hw, bias=None, act=ACT_NONE, alpha=0.0):
        N, Ho, Wo, O = dy.shape
        kh, kw, Cc, O2 = k.shape
        assert O2 == O
        H, W = in_hw
        pad_h = (Ho - 1) * stride + kh - H      # src/gpu/conv2d.cu:88-93
        pad_w = (Wo - 1) * stride + kw - W
        ddy, dk = self._up(dy, k)
        db = Buf.from_numpy(bias) if bias is not None else None
        out = Buf((N, H, W, Cc))
        check(self.lib.dh_conv2d_dx(ddy.ptr, dk.ptr, out.ptr, N, Ho, Wo, O, kh, kw, Cc, stride, stride,
                                    pad_h // 2, pad_w // 2, H, W, db.ptr if db else None, act, alpha,
                                    self.stream))
        return out.numpy()

    def conv2d_kernel_grad(self, dy, x, stride, pads, k_hw=None):
        N, Ho, Wo, O = dy.shape
        N2, H, W, Cc = x.shape
        assert N2 == N
        kh = H + pads[0] - stride * (Ho - 1)    # src/gpu/conv2d.cu:145-146
        kw = W + pads[1] - stride * (Wo - 1)
        if k_hw is not None:
            assert (kh, kw) == tuple(k_hw)
        dx_, ddy = self._up(x, dy)
        out = Buf((kh, kw, Cc, O))
        check(self.lib.dh_conv2d_dk(dx_.ptr, ddy.ptr, out.ptr, N, H, W, Cc, Ho, Wo, O, kh, kw, stride, stride,
                                    pads[0] // 2, pads[1] // 2, self.stream))
        return out.numpy()

    def conv2d_transpose(self, x, k, out_hw, stride, bias=None, act=ACT_NONE, alpha=0.0):
        # x [N,Hi,Wi,Ci], k [kh,kw,Co,Ci] -> y [N,Hout,Wout,Co]   (src/gpu/conv2d.cu:167-212)
        return self.conv2d_input_grad(x, k, stride, out_hw, bias, act, alpha)

    def conv2d_transpose_input_grad(self, dy, k, stride, in_hw):
        # forward conv of dy with pads re-derived from the extents (src/gpu/conv2d.cu:214-259)
        N, Hy, Wy, Co = dy.shape
        kh, kw = k.shape[:2]
        pads = ((in_hw[0] - 1) * stride + kh - Hy, (in_hw[1] - 1) * stride + kw - Wy)
        out = self.conv2d(dy, k, (stride, stride), pads)
        assert out.shape[1:3] == tuple(in_hw)
        return out

    def conv2d_transpose_kernel_grad(self, dy, x, stride, k_hw):
        # conv2d filter gradient with the activations' roles exchanged (src/gpu/conv2d.cu:264-307)
        Hy, Wy = dy.shape[1:3]
        Hi, Wi = x.shape[1:3]
        pads = ((Hi - 1) * stride + k_hw[0] - Hy, (Wi - 1) * stride + k_hw[1] - Wy)
        return self.conv2d_kernel_grad(x, dy, stride, pads, k_hw)

    # -- bias / activations --
    def bias_add(self, z, b):
        dz, db = self._up(z, b)
        out = Buf(z.shape)
        cols = z.shape[-1]
        check(self.lib.dh_bias_add(dz.ptr, db.ptr, out.ptr, z.size // cols, cols, self.stream))
        return out.numpy()

    def bias_grad(self, dz):
        d, = self._up(dz)
        cols = dz.shape[-1]
        out = Buf((cols,))
        check(self.lib.dh_bias_grad(d.ptr, out.ptr, dz.size // cols, cols, self.stream))
        return out.numpy()

    def act_bias_grad(self, act_ref, dout, act, alpha=0.0):
        r, d = self._up(act_ref, dout)
        cols = dout.shape[-1]
        dz, db = Buf(dout.shape), Buf((cols,))
        check(self.lib.dh_act_bias_grad(r.ptr, d.ptr, dz.ptr, db.ptr, dout.size // cols, cols, act, alpha,
                                        self.stream))
        return dz.numpy(), db.numpy()

    def bias_grad_parts(self, dz):
        """Row-range sums [parts, cols] whose sum over axis 0 (in dh_bias_grad's order) is the bias gradient."""
        d, = self._up(dz)
        cols = dz.shape[-1]
        parts = self.lib.dh_bias_grad_part_count(dz.size // cols, cols)
        out = Buf((parts, cols))
        check(self.lib.dh_bias_grad_parts(d.ptr, out.ptr, dz.size // cols, cols, self.stream))
        return out.numpy()

    def act_bias_grad_parts(self, act_ref, dout, act, alpha=0.0):
        r, d = self._up(act_ref, dout)
        cols = dout.shape[-1]
        parts = self.lib.dh_bias_grad_part_count(dout.size // cols, cols)
        dz, out = Buf(dout.shape), Buf((parts, cols))
        check(self.lib.dh_act_bias_grad_parts(r.ptr, d.ptr, dz.ptr, out.ptr, dout.size // cols, cols, act, alpha,
                                              self.stream))
        return dz.numpy(), out.numpy()

    def mat_sum_rows(self, a):
        d, = self._up(a)
        out = Buf((a.shape[0],))
        check(self.lib.dh_mat_sum_rows(d.ptr, out.ptr, a.shape[0], a.shape[1], self.stream))
        return out.numpy()

    def _unary(self, fn, a, *extra):
        a = np.ascontiguousarray(a, np.float32)
        d, = self._up(a)
        out = Buf(a.shape)
        check(fn(d.ptr, out.ptr, a.size, *extra, self.stream))
        return out.numpy()

    def _binary(self, fn, a, b, *extra_before_n):
        a, b = np.ascontiguousarray(a, np.float32), np.ascontiguousarray(b, np.float32)
        assert a.shape == b.shape
        da, db = self._up(a, b)
        out = Buf(a.shape)
        check(fn(da.ptr, db.ptr, out.ptr, *extra_before_n, a.size, self.stream))
        return out.numpy()

    def relu(self, a):
        return self._unary(self.lib.dh_relu, a)

    def relu_leaky(self, a, alpha=0.2):
        return self._unary(self.lib.dh_relu_leaky, a, alpha)

    def tanh(self, a):
        return self._unary(self.lib.dh_tanh, a)

    def sigmoid(self, a):
        return self._unary(self.lib.dh_sigmoid, a)

    def relu_grad(self, z, dout):
        return self._binary(self.lib.dh_relu_grad, z, dout)

    def leaky_relu_grad(self, z, dout, alpha):
        return self._binary(self.lib.dh_leaky_relu_grad, z, dout, alpha)

    def tanh_grad(self, t, dout):
        return self._binary(self.lib.dh_tanh_grad, t, dout)

    def sigmoid_grad(self, s, dout):
        return self._binary(self.lib.dh_sigmoid_grad, s, dout)

    def add(self, a, b):
        return self._binary(self.lib.dh_add, a, b)

    # -- losses --
    def sigmoid_cross_entropy(self, y, logits):
        dy, dl = self._up(y, logits)
        out = Buf((1,))
        check(self.lib.dh_sigmoid_cross_entropy(dy.ptr, dl.ptr, out.ptr, y.size, self.stream))
        return out.numpy()[0]

    def sigmoid_cross_entropy_grad(self, y, logits):
        return self._binary(self.lib.dh_sigmoid_cross_entropy_grad, y, logits)

    def mse(self, y, y_hat):
        dy, dh = self._up(y, y_hat)
        out = Buf((1,))
        check(self.lib.dh_mse(dy.ptr, dh.ptr, out.ptr, y.shape[0], y.size // y.shape[0], self.stream))
        return out.numpy()[0]

    def mse_grad(self, y, y_hat):
        return self._binary(self.lib.dh_mse_grad, y, y_hat)

    def argmax_acc(self, y, y_hat):
        dy, dh = self._up(y, y_hat)
        out = Buf((1,))
        check(self.lib.dh_argmax_acc(dy.ptr, dh.ptr, out.ptr, y.shape[0], y.shape[1], self.stream))
        return int(out.numpy()[0])

    # -- dense --
    def mm_mul(self, a, b):
        da, db = self._up(a, b)
        out = Buf((a.shape[0], b.shape[1]))
        check(self.lib.dh_gemm_nn(da.ptr, db.ptr, None, out.ptr, a.shape[0], a.shape[1], b.shape[1], self.stream))
        return out.numpy()

    def mat_mul_add(self, x, w, b):
        dx, dw, db = self._up(x, w, b)
        out = Buf((x.shape[0], w.shape[1]))
        check(self.lib.dh_gemm_nn(dx.ptr, dw.ptr, db.ptr, out.ptr, x.shape[0], x.shape[1], w.shape[1], self.stream))
        return out.numpy()

    def tmm_mul(self, a, b):
        da, db = self._up(a, b)
        out = Buf((a.shape[1], b.shape[1]))
        check(self.lib.dh_gemm_tn(da.ptr, db.ptr, out.ptr, a.shape[1], a.shape[0], b.shape[1], self.stream))
        return out.numpy()

    def mtm_mul(self, a, b):
        da, db = self._up(a, b)
        out = Buf((a.shape[0], b.shape[0]))
        check(self.lib.dh_gemm_nt(da.ptr, db.ptr, out.ptr, a.shape[0], a.shape[1], b.shape[0], self.stream))
        return out.numpy()

    # -- Adam --
    def moment_update(self, var, dv, a, b):
        dvar, ddv = self._up(var, dv)
        check(self.lib.dh_moment_update(dvar.ptr, ddv.ptr, a, b, dvar.size, self.stream))
        return dvar.numpy()

    def moment_update2(self, var, dv, a, b):
        dvar, ddv = self._up(var, dv)
        check(self.lib.dh_moment_update2(dvar.ptr, ddv.ptr, a, b, dvar.size, self.stream))
        return dvar.numpy()

    @staticmethod
    def adam_lrt(t, lr, beta1, beta2):
        """Host-side step size in float arithmetic (src/gpu/update.cu:81-96). Returns (t+1, lrt)."""
        f = np.float32
        t = f(f(t) + f(1))
        lrt = f(lr) * np.sqrt(f(1) - np.power(f(beta2), t, dtype=f), dtype=f) \
            / (f(1) - np.power(f(beta1), t, dtype=f))
        return t, f(lrt)

    def adam_apply(self, p, m, v, lrt, eps):
        dp, dm, dv = self._up(p, m, v)
        check(self.lib.dh_adam_update(dp.ptr, dm.ptr, dv.ptr, lrt, eps, dp.size, self.stream))
        return dp.numpy()

    def adam_step(self, p, m, v, g, beta1, beta2, lrt, eps):
        dp, dm, dv, dg = self._up(p, m, v, g)
        one = np.float32(1)
        check(self.lib.dh_adam_step(dp.ptr, dm.ptr, dv.ptr, dg.ptr, beta1, one - np.float32(beta1), beta2,
                                    one - np.float32(beta2), lrt, eps, dp.size, self.stream))
        return dp.numpy(), dm.numpy(), dv.numpy()

    def adam_step_multi(self, items, beta1, beta2, eps):
        """items: [(p, m, v, g1, g2 or None, lrt)] -> [(p, m, v)] after one step, all in one launch.
        A gradient with one more axis than p is taken as row-range sums [parts, n] (see bias_grad_parts)."""
        arr = (AdamItem * len(items))()
        bufs = []
        for i, (p, m, v, g1, g2, lrt) in enumerate(items):
            dp, dm, dv, dg = self._up(p, m, v, g1)
            dh = Buf.from_numpy(g2) if g2 is not None else None
            bufs.append((dp, dm, dv, dg, dh))
            parts = [g.shape[0] if g is not None and g.ndim == p.ndim + 1 else 0 for g in (g1, g2)]
            arr[i] = AdamItem(dp.ptr, dm.ptr, dv.ptr, dg.ptr, dh.ptr if dh else None, dp.size, lrt, parts[0], parts[1])
        one = np.float32(1)
        check(self.lib.dh_adam_step_multi(arr, len(items), beta1, one - np.float32(beta1), beta2,
                                          one - np.float32(beta2), eps, self.stream))
        return [(b[0].numpy(), b[1].numpy(), b[2].numpy()) for b in bufs]

    def vect_update(self, var, dv, coeff):
        dvar, ddv, dc = self._up(var, dv, np.array([coeff], np.float32))
        check(self.lib.dh_sgd_update(dvar.ptr, ddv.ptr, dc.ptr, dvar.size, self.stream))
        return dvar.numpy()

"""ctypes binding of the host library's C facade (host/dcgan.hh): the reference's DCGAN built on
the operator graph.  The program mode is process-wide and read once from RT_MODE, so choose it
before creating a model:

    m = DcganModel(batch=64, seed=1, mode="GPU")        # HIP backend
    m = DcganModel(batch=2, seed=1, mode="CPU", cpu_backend=".../liboracle_backend.so")   # tests only

In a CPU mode a backend library exporting orc_register_backend() must be supplied -- the host
library itself holds the HIP backend only.
"""
import ctypes as C
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libdcgan_host.so")

_lib = None
_fp = C.POINTER(C.c_float)


def load():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is not built; run `python dcgan-cuda_amd/build.py`" % LIB_PATH)
        lib = C.CDLL(LIB_PATH, mode=C.RTLD_GLOBAL)
        lib.dg_last_error.restype = C.c_char_p
        lib.dg_create.restype = C.c_void_p
        lib.dg_create.argtypes = [C.c_int, C.c_ulonglong]
        lib.dg_destroy.argtypes = [C.c_void_p]
        lib.dg_set_fusion.argtypes = [C.c_int]
        lib.dg_set_pairing.argtypes = [C.c_int]
        lib.dg_set_name_results.argtypes = [C.c_int]
        lib.dg_set_labels.argtypes = [C.c_void_p, _fp]
        lib.dg_disc_pass.argtypes = [C.c_void_p, _fp]
        lib.dg_num_vars.argtypes = [C.c_void_p]
        lib.dg_var_size.argtypes = [C.c_void_p, C.c_int]
        lib.dg_var_size.restype = C.c_long
        lib.dg_var_read.argtypes = [C.c_void_p, C.c_int, _fp]
        lib.dg_var_write.argtypes = [C.c_void_p, C.c_int, _fp]
        lib.dg_set_inputs.argtypes = [C.c_void_p, _fp, _fp]
        lib.dg_d_step.argtypes = [C.c_void_p, _fp]
        lib.dg_g_step.argtypes = [C.c_void_p, _fp]
        lib.dg_d_step_fed.argtypes = [C.c_void_p, _fp, _fp, _fp]
        lib.dg_g_step_fed.argtypes = [C.c_void_p, _fp, _fp]
        lib.dg_generate.argtypes = [C.c_void_p, _fp]
        lib.dg_eval.argtypes = [C.c_void_p, C.c_char_p, _fp, C.POINTER(C.c_long)]
        lib.dg_eval_many.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(_fp), C.c_int]
        lib.dg_last_schedule_size.argtypes = [C.c_void_p]
        lib.dg_last_launch_count.argtypes = [C.c_void_p]
        for name in ("dg_save_vars", "dg_load_vars", "dg_save_state", "dg_load_state"):
            getattr(lib, name).argtypes = [C.c_void_p, C.c_char_p]
        lib.dg_npz_inspect.argtypes = [C.c_char_p, C.POINTER(C.c_long), C.POINTER(C.c_long)]
        lib.dg_images_normalize.argtypes = [C.c_char_p, C.c_long, _fp]
        lib.dg_images_load.argtypes = [C.c_char_p, C.c_long, C.c_long, _fp]
        lib.dg_images_save_samples.argtypes = [_fp, C.c_long, C.c_long, C.c_char_p]
        _lib = lib
    return _lib


class HostError(RuntimeError):
    pass


def _check(rc):
    if rc != 0:
        raise HostError(load().dg_last_error().decode())


def _p(a):
    return a.ctypes.data_as(_fp)


# variable order of the facade: g conv-transpose 1..4 (w,b), g dense (w,b), d conv 0..3 (w,b), d dense (w,b)
VAR_NAMES = ["g1_w", "g1_b", "g2_w", "g2_b", "g3_w", "g3_b", "g4_w", "g4_b", "g0_w", "g0_b",
             "d0_w", "d0_b", "d1_w", "d1_b", "d2_w", "d2_b", "d3_w", "d3_b", "d4_w", "d4_b"]


def var_shapes():
    return {"g1_w": (5, 5, 256, 512), "g1_b": (256,), "g2_w": (5, 5, 128, 256), "g2_b": (128,),
            "g3_w": (5, 5, 64, 128), "g3_b": (64,), "g4_w": (5, 5, 3, 64), "g4_b": (3,),
            "g0_w": (100, 8192), "g0_b": (8192,),
            "d0_w": (5, 5, 3, 64), "d0_b": (64,), "d1_w": (5, 5, 64, 128), "d1_b": (128,),
            "d2_w": (5, 5, 128, 256), "d2_b": (256,), "d3_w": (5, 5, 256, 512), "d3_b": (512,),
            "d4_w": (8192, 1), "d4_b": (1,)}


class DcganModel:
    def __init__(self, batch, seed=1, mode="GPU", cpu_backend=None):
        want = {"GPU": "GPU", "CPU": "CPU", "MCPU": "MCPU"}[mode]
        have = os.environ.get("RT_MODE")
        if have is not None and have != want and getattr(DcganModel, "_mode_used", None):
            raise HostError("the program mode is fixed for the life of the process (RT_MODE=%s)" % have)
        os.environ["RT_MODE"] = want
        DcganModel._mode_used = want
        self.lib = load()
        if mode != "GPU":
            if cpu_backend is None:
                raise HostError("a CPU mode needs a backend library (the host library holds the HIP backend only)")
            self._backend = C.CDLL(cpu_backend, mode=C.RTLD_GLOBAL)
            # a library named *_f64.so registers the float64-accumulating flavour of the oracle
            reg = "orc_register_backend_f64" if cpu_backend.endswith("_f64.so") else "orc_register_backend"
            getattr(self._backend, reg)()
        self.batch = batch
        self.h = self.lib.dg_create(batch, seed)
        if not self.h:
            raise HostError(self.lib.dg_last_error().decode())

    def close(self):
        if self.h:
            self.lib.dg_destroy(self.h)
            self.h = None

    def set_fusion(self, on):
        self.lib.dg_set_fusion(1 if on else 0)

    def set_name_results(self, on):
        """Off: a run hands the backend the instruction list and nothing else, as the reference's
        Graph::run does (src/ops/graph.cu:194-200); every intermediate tensor is then kept.  On (default):
        the run names the tensors it reads back and the planner may leave out the others."""
        self.lib.dg_set_name_results(1 if on else 0)

    def set_pairing(self, on):
        """With fusion: run same-filter convolutions of the two discriminator towers as one launch."""
        self.lib.dg_set_pairing(1 if on else 0)

    def num_vars(self):
        return self.lib.dg_num_vars(self.h)

    def var(self, name):
        i = VAR_NAMES.index(name)
        out = np.empty(self.lib.dg_var_size(self.h, i), np.float32)
        _check(self.lib.dg_var_read(self.h, i, _p(out)))
        return out.reshape(var_shapes()[name])

    def set_var(self, name, value):
        i = VAR_NAMES.index(name)
        a = np.ascontiguousarray(value, np.float32)
        assert a.size == self.lib.dg_var_size(self.h, i), name
        _check(self.lib.dg_var_write(self.h, i, _p(a)))

    def set_inputs(self, z=None, x=None):
        z = None if z is None else np.ascontiguousarray(z, np.float32)
        x = None if x is None else np.ascontiguousarray(x, np.float32)
        _check(self.lib.dg_set_inputs(self.h, _p(z) if z is not None else None, _p(x) if x is not None else None))

    def d_step(self, want_loss=True, z=None, x=None):
        """One discriminator step; z / x (host arrays) are fed to the run itself when given."""
        loss = C.c_float()
        z = None if z is None else np.ascontiguousarray(z, np.float32)
        x = None if x is None else np.ascontiguousarray(x, np.float32)
        _check(self.lib.dg_d_step_fed(self.h, None if z is None else _p(z), None if x is None else _p(x),
                                      C.byref(loss) if want_loss else None))
        return loss.value if want_loss else None

    def g_step(self, want_loss=True, z=None):
        loss = C.c_float()
        z = None if z is None else np.ascontiguousarray(z, np.float32)
        _check(self.lib.dg_g_step_fed(self.h, None if z is None else _p(z), C.byref(loss) if want_loss else None))
        return loss.value if want_loss else None

    def set_labels(self, y):
        """Labels [batch, 1] of the stand-alone discriminator pass."""
        y = np.ascontiguousarray(y, np.float32)
        assert y.size == self.batch
        _check(self.lib.dg_set_labels(self.h, _p(y)))

    def disc_pass(self, want_loss=True):
        """The discriminator alone on the resident images and labels: loss, the gradients of all ten
        discriminator variables and of the images, one run (names: disc_loss, grad:disc_loss:<var>,
        grad:disc_loss:x_real)."""
        loss = C.c_float()
        _check(self.lib.dg_disc_pass(self.h, C.byref(loss) if want_loss else None))
        return loss.value if want_loss else None

    def sync(self):
        _check(self.lib.dg_sync())

    def generate(self, to_host=True):
        """Generator forward pass.  to_host=False leaves the images on the device and does not wait."""
        if not to_host:
            _check(self.lib.dg_generate(self.h, None))
            return None
        out = np.empty((self.batch, 64, 64, 3), np.float32)
        _check(self.lib.dg_generate(self.h, _p(out)))
        return out

    def eval(self, what, shape=None):
        n = C.c_long()
        _check(self.lib.dg_eval(self.h, what.encode(), None, C.byref(n)))
        out = np.empty(max(n.value, 1), np.float32)
        _check(self.lib.dg_eval(self.h, what.encode(), _p(out), None))
        return out.reshape(shape) if shape is not None else out

    def eval_many(self, names):
        """Several named tensors from ONE run of the graph: {name: flat float32 array}."""
        outs = []
        for what in names:
            n = C.c_long()
            _check(self.lib.dg_eval(self.h, what.encode(), None, C.byref(n)))
            outs.append(np.empty(max(n.value, 1), np.float32))
        ptrs = (_fp * len(outs))(*[_p(a) for a in outs])
        _check(self.lib.dg_eval_many(self.h, ";".join(names).encode(), ptrs, len(outs)))
        return dict(zip(names, outs))

    @staticmethod
    def grad_name(loss, name):
        return "grad:%s:%s" % (loss, name if name in ("x_fake", "x_real") else VAR_NAMES.index(name))

    def grad(self, loss, name):
        if name == "x_fake":
            return self.eval("grad:%s:x_fake" % loss, (self.batch, 64, 64, 3))
        return self.eval("grad:%s:%d" % (loss, VAR_NAMES.index(name)), var_shapes()[name])

    def last_schedule_size(self):
        return self.lib.dg_last_schedule_size(self.h)

    def last_launch_count(self):
        """Steps (single or fused launches) the last run on the HIP backend issued."""
        return self.lib.dg_last_launch_count(self.h)

    def save_vars(self, path):
        """Trainable variables, creation order; numpy .npz (arr_0, arr_1, ...) when path ends in .npz."""
        _check(self.lib.dg_save_vars(self.h, path.encode()))

    def load_vars(self, path):
        _check(self.lib.dg_load_vars(self.h, path.encode()))

    def save_state(self, path):
        """All variables, the Adam moments and step counters (.npz): enough to continue training."""
        _check(self.lib.dg_save_state(self.h, path.encode()))

    def load_state(self, path):
        _check(self.lib.dg_load_state(self.h, path.encode()))


def npz_inspect(path):
    """(arrays, elements) of a .npz archive as the library's own reader sees it; HostError if it refuses the file."""
    a, n = C.c_long(), C.c_long()
    _check(load().dg_npz_inspect(path.encode(), C.byref(a), C.byref(n)))
    return a.value, n.value


def images_normalize(pix):
    """uint8 array -> float32 array of the same shape, pix / 127.5 - 1 (src/datasets/celeba.cu:27-28)."""
    pix = np.ascontiguousarray(pix, dtype=np.uint8)
    out = np.empty(pix.shape, np.float32)
    _check(load().dg_images_normalize(pix.ctypes.data_as(C.c_char_p), pix.size, _p(out)))
    return out


def images_load(directory, idx_beg, idx_end):
    """<directory>/<6-digit index>.ppm for idx_beg <= index < idx_end -> [n, 64, 64, 3] in [-1, 1]."""
    out = np.empty((idx_end - idx_beg, 64, 64, 3), np.float32)
    _check(load().dg_images_load(directory.encode(), idx_beg, idx_end, _p(out)))
    return out


def images_save_samples(data, width, height, path):
    """width x height images [n, 64, 64, 3] in [-1, 1] -> one PPM mosaic (src/datasets/celeba.cu:44-68)."""
    data = np.ascontiguousarray(data, dtype=np.float32)
    assert data.size == width * height * 64 * 64 * 3
    _check(load().dg_images_save_samples(_p(data), width, height, path.encode()))

"""ctypes front-end of oracle/_ref/libseam_ref.so (test infrastructure): instructions made by the
REFERENCE's rt::Node::op_* factories (src/runtime/node.cu:118-294 and the element-wise ones around
them), run through the reference's CPU kernel table on host buffers and through this build's HIP kernel
table -- dcgan-cuda_amd/host/hip_table.cc compiled against the reference's src/runtime/node.hh -- on
device buffers."""
import ctypes as C
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "oracle", "_ref", "libseam_ref.so")
_fp = C.POINTER(C.c_float)
_lib = None


def have():
    return os.path.exists(LIB)


def load():
    global _lib
    if _lib is None:
        lib = C.CDLL(LIB)
        lib.seam_last_error.restype = C.c_char_p
        lib.seam_node_new.restype = C.c_void_p
        lib.seam_node_new.argtypes = [C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int), C.POINTER(C.c_float)]
        for name in ("seam_node_type", "seam_node_free", "seam_run_cpu", "seam_run_hip"):
            getattr(lib, name).argtypes = [C.c_void_p]
        lib.seam_node_layout.argtypes = [C.POINTER(C.c_ulong), C.c_int]
        _lib = lib
    return _lib


def layout(fn):
    buf = (C.c_ulong * 32)()
    n = fn(buf, 32)
    return list(buf)[:n]


def node(op, tensors, ints=(), floats=()):
    """tensors: five addresses (in1, in2, in3, out1, out2 in the factory's roles), 0 for unused."""
    lib = load()
    t = (C.c_void_p * 5)(*[C.c_void_p(int(a)) if a else None for a in tensors])
    i = (C.c_int * max(len(ints), 1))(*[int(v) for v in ints])
    f = (C.c_float * max(len(floats), 1))(*[float(v) for v in floats])
    h = lib.seam_node_new(op.encode(), t, i, f)
    if not h:
        raise KeyError("no reference factory bound for " + op)
    return C.c_void_p(h)


def run_both(A, op, arrays, ints=(), floats=(), host_slots=()):
    """arrays: five numpy float32 arrays or None (in1, in2, in3, out1, out2); out1 (and out2) are
    read back after the run.  host_slots: slots whose pointer is a HOST pointer on both backends (the
    Adam step counter).  Returns ((cpu out1, cpu out2), (hip out1, hip out2), op code)."""
    lib = load()
    cpu = [None if a is None else np.array(a, dtype=np.float32, order="C") for a in arrays]
    n = node(op, [0 if a is None else a.ctypes.data for a in cpu], ints, floats)
    code = lib.seam_node_type(n)
    try:
        if lib.seam_run_cpu(n) != 0:
            raise RuntimeError(lib.seam_last_error().decode())
    finally:
        lib.seam_node_free(n)
    host = [None if a is None else np.array(a, dtype=np.float32, order="C") for a in arrays]
    dev = [None if (a is None or s in host_slots) else A.Buf.from_numpy(a) for s, a in enumerate(host)]
    ptrs = [0 if a is None else (a.ctypes.data if s in host_slots else dev[s].ptr) for s, a in enumerate(host)]
    n = node(op, ptrs, ints, floats)
    try:
        if lib.seam_run_hip(n) != 0:
            raise RuntimeError(lib.seam_last_error().decode())
    finally:
        lib.seam_node_free(n)
    got = [None if a is None else (a if s in host_slots else dev[s].numpy()) for s, a in enumerate(host)]
    return (cpu[3], cpu[4]), (got[3], got[4]), code


def run_hip(A, op, arrays, ints=(), floats=()):
    """As run_both, the HIP table only: returns out1 (for shapes where the reference's CPU loops take minutes)."""
    lib = load()
    host = [None if a is None else np.array(a, dtype=np.float32, order="C") for a in arrays]
    dev = [None if a is None else A.Buf.from_numpy(a) for a in host]
    n = node(op, [0 if d is None else d.ptr for d in dev], ints, floats)
    try:
        if lib.seam_run_hip(n) != 0:
            raise RuntimeError(lib.seam_last_error().decode())
    finally:
        lib.seam_node_free(n)
    return dev[3].numpy()


class Program:
    """An instruction graph held by the REFERENCE's rt::Graph (src/runtime/graph.cu): instructions come
    from the reference's factories with explicit predecessors, the execution order from the reference's
    topological_sort, and the list runs through the reference's CPU table or through hip::run -- the
    planning runner compiled against the reference's node.hh / nodes-list.hh."""

    def __init__(self):
        lib = load()
        lib.seam_prog_new.restype = C.c_void_p
        lib.seam_prog_free.argtypes = [C.c_void_p]
        lib.seam_prog_add.argtypes = [C.c_void_p, C.c_char_p, C.POINTER(C.c_void_p), C.POINTER(C.c_int),
                                      C.POINTER(C.c_float), C.POINTER(C.c_int), C.c_int]
        lib.seam_prog_order.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.POINTER(C.c_int), C.c_int]
        lib.seam_prog_run_cpu.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int]
        lib.seam_prog_run_hip.argtypes = [C.c_void_p, C.POINTER(C.c_int), C.c_int, C.c_int, C.c_int,
                                          C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_int)]
        self.lib = lib
        self.h = C.c_void_p(lib.seam_prog_new())
        self.count = 0

    def close(self):
        if self.h:
            self.lib.seam_prog_free(self.h)
            self.h = None

    def add(self, op, tensors, ints=(), floats=(), preds=()):
        """tensors: five addresses as for node(); preds: ids of the instructions this one waits for."""
        t = (C.c_void_p * 5)(*[C.c_void_p(int(a)) if a else None for a in tensors])
        i = (C.c_int * max(len(ints), 1))(*[int(v) for v in ints])
        f = (C.c_float * max(len(floats), 1))(*[float(v) for v in floats])
        p = (C.c_int * max(len(preds), 1))(*[int(v) for v in preds])
        nid = self.lib.seam_prog_add(self.h, op.encode(), t, i, f, p, len(preds))
        if nid < 0:
            raise KeyError("no reference factory bound for " + op)
        self.count += 1
        return nid

    @staticmethod
    def _ids(want):
        return (C.c_int * max(len(want), 1))(*[int(v) for v in want]), len(want)

    def order(self, want):
        w, n = self._ids(want)
        ids = (C.c_int * (self.count + 1))()
        got = self.lib.seam_prog_order(self.h, w, n, ids, self.count + 1)
        return list(ids)[:got]

    def run_cpu(self, want):
        w, n = self._ids(want)
        if self.lib.seam_prog_run_cpu(self.h, w, n) != 0:
            raise RuntimeError(self.lib.seam_last_error().decode())

    def run_hip(self, want, fuse=True, pair=True, keep=None):
        """keep=None: nothing is said about the tensors read afterwards (gpu::run's own signature);
        otherwise the addresses handed to hip::set_protected_tensors.  Returns the launch count."""
        w, n = self._ids(want)
        launches = C.c_int(0)
        if keep is None:
            k, nk = (C.c_void_p * 1)(), -1
        else:
            k, nk = (C.c_void_p * max(len(keep), 1))(*[C.c_void_p(int(a)) for a in keep]), len(keep)
        if self.lib.seam_prog_run_hip(self.h, w, n, int(fuse), int(pair), k, nk, C.byref(launches)) != 0:
            raise RuntimeError(self.lib.seam_last_error().decode())
        return launches.value

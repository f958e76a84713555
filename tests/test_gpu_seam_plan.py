"""The fusing and pairing runner behind the reference's own seam.  dcgan-cuda_amd/host/hip_kernels.cc is
compiled -- unchanged -- against the reference's src/runtime/node.hh and nodes-list.hh; the instruction
graph of a discriminator-style optimiser step (two towers that share their filters: conv2d ->
mat_rvect_add -> relu_leaky twice, a dense head, sigmoid cross-entropy, every gradient, the `add` nodes
that join the towers' gradients, and moment_update / moment_update2 / adam_update per variable) is made
by the reference's rt::Node::op_* factories inside the reference's rt::Graph and ordered by its
topological_sort, exactly as src/ops/graph.cu:194-200 hands a list to gpu::run.  The list then runs
through hip::run and, node by node, through the reference's cpu::kernels_list, and the tensors are
compared.

Two callers are covered.  One that hands over nothing but the list (gpu::run's own signature,
src/gpu/runner.cu:10): every tensor of every node must then hold the reference's value after the run.
One that names the tensors it reads back (hip::set_protected_tensors, the one call a fused drop-in adds
to src/ops/graph.cu): those tensors, the variables and the moments must hold the reference's values and
the plan must be shorter."""
import numpy as np
import pytest

import seam
from common import RTOL, ATOL, same_pad

pytestmark = pytest.mark.gpu

ALPHA = 0.2
LR, B1, B2, EPS = 2e-4, 0.5, 0.999, 1e-8


@pytest.fixture(scope="module")
def A():
    if not seam.have():
        pytest.fail("oracle/_ref/libseam_ref.so is missing: build() makes it where the reference tree is mounted")
    import __graft_entry__ as ge
    return ge.load_package().hipabi


class Host:
    """Tensors of the reference's CPU run: numpy arrays."""

    def __init__(self):
        self.t = {}

    def put(self, name, a):
        self.t[name] = np.array(a, dtype=np.float32, order="C")
        return self.t[name].ctypes.data

    def host(self, name, a):
        return self.put(name, a)

    def get(self, name):
        return self.t[name]


class Device:
    """Tensors of the HIP run: device buffers, except those the instruction set keeps on the host (Adam's
    step counter, src/gpu/update.cu:81-96)."""

    def __init__(self, A):
        self.A, self.t, self.h = A, {}, {}

    def put(self, name, a):
        self.t[name] = self.A.Buf.from_numpy(np.array(a, dtype=np.float32))
        return self.t[name].ptr

    def host(self, name, a):
        self.h[name] = np.array(a, dtype=np.float32, order="C")
        return self.h[name].ctypes.data

    def get(self, name):
        return self.h[name] if name in self.h else self.t[name].numpy()


def build_step(mem, N, H, C0, C1, C2, seed):
    """Returns (program, ids of the instructions a caller would ask for, names of all tensors written,
    names of the variables and moments).  Same seed -> same values in every memory."""
    rng = np.random.default_rng(seed)
    P = seam.Program()
    s, k = 2, 5
    (p1, H1), (p2, H2) = same_pad(H, k, s), same_pad(-(-H // s), k, s)
    F = H2 * H2 * C2
    z = lambda *shape: np.zeros(shape, np.float32)
    u = lambda *shape: rng.uniform(-1, 1, shape).astype(np.float32)
    var = {"k1": u(k, k, C0, C1) * 0.05, "b1": u(C1) * 0.1, "k2": u(k, k, C1, C2) * 0.05, "b2": u(C2) * 0.1,
           "w": u(F, 1) * 0.05, "bw": u(1) * 0.1}
    ptr, state = {}, []
    for name, a in var.items():
        ptr[name] = mem.put(name, a)
        ptr["m_" + name] = mem.put("m_" + name, u(*a.shape) * 0.1)
        ptr["v_" + name] = mem.put("v_" + name, np.abs(u(*a.shape)) * 0.01 + 1e-3)
        ptr["t_" + name] = mem.host("t_" + name, [3.0])
        state += [name, "m_" + name, "v_" + name, "t_" + name]
    written = []

    def out(name, *shape):
        ptr[name] = mem.put(name, z(*shape))
        written.append(name)
        return ptr[name]

    grads = {name: [] for name in var}      # (tensor name, producing instruction) per tower
    readers = {name: [] for name in var}    # instructions that read the variable
    losses = []
    for tower, label in (("r", 1.0), ("f", 0.0)):
        T = lambda name: name + "_" + tower
        x = mem.put(T("x"), u(N, H, H, C0))
        y = mem.put(T("y"), np.full((N, 1), label, np.float32))
        # forward: src/api/layers.cu:85-92 lowers conv2d + bias to conv2d -> mat_rvect_add
        c1 = P.add("conv2d", [x, ptr["k1"], 0, out(T("c1"), N, H1, H1, C1), 0], [s, s, p1, p1, N, H, H, C0, k, k, C0, C1])
        n1 = N * H1 * H1
        z1 = P.add("mat_rvect_add", [ptr[T("c1")], ptr["b1"], 0, out(T("z1"), n1, C1), 0], [n1, C1], preds=[c1])
        a1 = P.add("relu_leaky", [ptr[T("z1")], 0, 0, out(T("a1"), n1, C1), 0], [n1 * C1], [ALPHA], preds=[z1])
        c2 = P.add("conv2d", [ptr[T("a1")], ptr["k2"], 0, out(T("c2"), N, H2, H2, C2), 0],
                   [s, s, p2, p2, N, H1, H1, C1, k, k, C1, C2], preds=[a1])
        n2 = N * H2 * H2
        z2 = P.add("mat_rvect_add", [ptr[T("c2")], ptr["b2"], 0, out(T("z2"), n2, C2), 0], [n2, C2], preds=[c2])
        a2 = P.add("relu_leaky", [ptr[T("z2")], 0, 0, out(T("a2"), n2, C2), 0], [n2 * C2], [ALPHA], preds=[z2])
        lg = P.add("mat_mul_add", [ptr[T("a2")], ptr["w"], ptr["bw"], out(T("logits"), N, 1), 0], [N, F, 1], preds=[a2])
        ls = P.add("sigmoid_cross_entropy", [y, ptr[T("logits")], 0, out(T("loss"), 1), 0], [N], preds=[lg])
        losses.append((T("loss"), ls))
        # backward
        dl = P.add("sigmoid_cross_entropy_grad", [y, ptr[T("logits")], 0, out(T("dlogits"), N, 1), 0], [N], preds=[lg])
        dw = P.add("tmat_mat_mul", [ptr[T("a2")], ptr[T("dlogits")], 0, out(T("dw"), F, 1), 0], [F, N, 1], preds=[a2, dl])
        dbw = P.add("mat_sum_cols", [ptr[T("dlogits")], 0, 0, out(T("dbw"), 1), 0], [N, 1], preds=[dl])
        da2 = P.add("mat_tmat_mul", [ptr[T("dlogits")], ptr["w"], 0, out(T("da2"), N, F), 0], [N, 1, F], preds=[dl])
        dz2 = P.add("leaky_relu_grad", [ptr[T("z2")], ptr[T("da2")], 0, out(T("dz2"), n2, C2), 0], [n2 * C2], [ALPHA],
                    preds=[z2, da2])
        db2 = P.add("mat_sum_cols", [ptr[T("dz2")], 0, 0, out(T("db2"), C2), 0], [n2, C2], preds=[dz2])
        dk2 = P.add("conv2d_kernel_grad", [ptr[T("dz2")], ptr[T("a1")], 0, out(T("dk2"), k, k, C1, C2), 0],
                    [s, s, N, H2, H2, C2, N, H1, H1, C1, p2, p2], preds=[dz2, a1])
        da1 = P.add("conv2d_input_grad", [ptr[T("dz2")], ptr["k2"], 0, out(T("da1"), N, H1, H1, C1), 0],
                    [s, s, N, H2, H2, C2, k, k, C1, C2, N, H1, H1, C1], preds=[dz2])
        dz1 = P.add("leaky_relu_grad", [ptr[T("z1")], ptr[T("da1")], 0, out(T("dz1"), n1, C1), 0], [n1 * C1], [ALPHA],
                    preds=[z1, da1])
        db1 = P.add("mat_sum_cols", [ptr[T("dz1")], 0, 0, out(T("db1"), C1), 0], [n1, C1], preds=[dz1])
        dk1 = P.add("conv2d_kernel_grad", [ptr[T("dz1")], x, 0, out(T("dk1"), k, k, C0, C1), 0],
                    [s, s, N, H1, H1, C1, N, H, H, C0, p1, p1], preds=[dz1])
        for name, node in (("w", dw), ("bw", dbw), ("k2", dk2), ("b2", db2), ("k1", dk1), ("b1", db1)):
            grads[name].append((T("d" + name), node))
        for name, nodes in (("k1", [c1]), ("b1", [z1]), ("k2", [c2, da1]), ("b2", [z2]), ("w", [lg, da2]), ("bw", [lg])):
            readers[name] += nodes
    loss = P.add("add", [ptr[losses[0][0]], ptr[losses[1][0]], 0, out("loss", 1), 0], [1], preds=[losses[0][1], losses[1][1]])
    steps = []
    for name, a in var.items():
        n = a.size
        (ga, na), (gb, nb) = grads[name]
        g = P.add("add", [ptr[ga], ptr[gb], 0, out("g_" + name, n), 0], [n], preds=[na, nb])
        m1 = P.add("moment_update", [ptr["g_" + name], 0, 0, ptr["m_" + name], 0], [n], [B1, 1 - B1], preds=[g])
        m2 = P.add("moment_update2", [ptr["g_" + name], 0, 0, ptr["v_" + name], 0], [n], [B2, 1 - B2], preds=[g])
        # The reference's sort breaks ties by node address (std::set<Node*>, src/runtime/graph.cu:47-75), so
        # the order differs from one build of the graph to the next: the in-place update also waits for
        # every instruction that reads the variable, which makes the step's result independent of it.
        steps.append(P.add("adam_update", [ptr["m_" + name], ptr["v_" + name], 0, ptr[name], ptr["t_" + name]], [n],
                           [LR, B1, B2, EPS], preds=[m1, m2] + readers[name]))
    return P, [loss] + steps, written, state, ptr


def close(got, exp, what):
    scale = max(1.0, float(np.abs(exp).max()))
    np.testing.assert_allclose(got, exp, rtol=RTOL, atol=ATOL * scale, err_msg=what)


SHAPES = [  # batch, image extent, channels of the input and of the two layers
    (16, 16, 16, 32, 64),      # buffer-load kernels, paired launches
    (4, 12, 3, 8, 16),         # 3-channel image layer, general kernels
]


@pytest.mark.parametrize("shape", SHAPES)
def test_optimiser_step_through_the_reference_seam(A, shape):
    seed = 100 + sum(shape)
    cpu = Host()
    P, want, written, state, _ = build_step(cpu, *shape, seed)
    order = P.order(want)
    assert len(order) == P.count, "the reference's sort must reach every instruction of the step"
    P.run_cpu(want)
    P.close()

    counts = {}
    # (fusion, pairing, names handed to set_protected_tensors or None) -> which tensors must agree
    for mode, fuse, pair, keep in (("table", False, False, None), ("list only", True, True, None),
                                   ("list only, unpaired", True, False, None), ("results named", True, True, ["loss"])):
        print("seam plan", shape, mode, flush=True)
        dev = Device(A)
        Pd, want_d, written_d, state_d, ptr = build_step(dev, *shape, seed)
        assert sorted(Pd.order(want_d)) == sorted(order)
        counts[mode] = Pd.run_hip(want_d, fuse, pair, None if keep is None else [ptr[n] for n in keep])
        check = state + (written if keep is None else keep)
        for name in check:
            close(dev.get(name), cpu.get(name), "%s: %s" % (mode, name))
        Pd.close()
    for name in state:
        if name.startswith("t_"):
            assert cpu.get(name)[0] == 4.0      # every backend advanced its own copy of the step counter once
    print("launches", counts, flush=True)
    assert counts["table"] == len(order)
    # a caller that says nothing still gets the fusions that lose no tensor ...
    assert counts["list only"] < counts["table"]
    assert counts["list only"] <= counts["list only, unpaired"]
    # ... and one that names what it reads gets the short plan
    assert counts["results named"] < counts["list only"]


def test_unnamed_intermediate_results_are_not_lost(A):
    """The conv2d output and the pre-activation of a fused layer, and a bias gradient that only the
    optimiser reads, exist after a run whose caller named nothing -- and are really left out (stay as
    initialised) once the caller has named its results, which is what makes naming them necessary."""
    shape = SHAPES[0]
    cpu = Host()
    P, want, written, state, _ = build_step(cpu, *shape, 7)
    P.run_cpu(want)
    P.close()
    dev = Device(A)
    Pd, want_d, _, _, ptr = build_step(dev, *shape, 7)
    Pd.run_hip(want_d, True, True, None)
    for name in ("c1_r", "z1_f", "c2_f", "db2_r", "g_k1", "dk1_f"):
        close(dev.get(name), cpu.get(name), name)
    Pd.close()
    dev = Device(A)
    Pd, want_d, _, _, ptr = build_step(dev, *shape, 7)
    Pd.run_hip(want_d, True, True, [ptr["loss"]])
    left_out = [name for name in ("c1_r", "z1_f", "c2_f", "db2_r", "g_k1") if not dev.get(name).any()]
    assert left_out, "the short plan is expected to skip intermediate tensors"
    close(dev.get("loss"), cpu.get("loss"), "loss")
    Pd.close()

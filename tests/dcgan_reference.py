"""Helpers for the whole-network tests: seeded synthetic weights/inputs, a float64 torch restatement
of the reference DCGAN (dcgan/main.cu:89-120, :217-249, :304-307) used to pin the operator graph's
differentiation, and a script mode that evaluates the network through the host library in
RT_MODE=CPU (the oracle as backend) and dumps everything to an .npz for the GPU parity test.

    python tests/dcgan_reference.py <batch> <seed> <out.npz> [<iterations> [f64]]
    python tests/dcgan_reference.py <batch> <seed> <out.npz> disc [f64]     (the discriminator pass alone)
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

G_VARS = ["g1_w", "g1_b", "g2_w", "g2_b", "g3_w", "g3_b", "g4_w", "g4_b", "g0_w", "g0_b"]
D_VARS = ["d0_w", "d0_b", "d1_w", "d1_b", "d2_w", "d2_b", "d3_w", "d3_b", "d4_w", "d4_b"]


def synthetic(batch, seed, shapes):
    """Weights ~ N(0, 0.02) (the generator's dense weight too, so that activations stay O(1)),
    small non-zero biases so that bias paths are exercised, z and images ~ U(-1, 1)."""
    rng = np.random.default_rng(seed)
    w = {}
    for name, shape in shapes.items():
        scale = 0.02 if name.endswith("_w") else 0.01
        w[name] = (rng.standard_normal(shape) * scale).astype(np.float32)
    z = rng.uniform(-1, 1, (batch, 100)).astype(np.float32)
    x = rng.uniform(-1, 1, (batch, 64, 64, 3)).astype(np.float32)
    return w, z, x


def labels(batch, seed):
    """Random 0/1 labels [batch, 1] of the stand-alone discriminator pass (Bernoulli 1/2)."""
    return (np.random.default_rng(seed + 1000).random((batch, 1)) < 0.5).astype(np.float32)


def disc_names():
    """(key in the dump, facade name) of the discriminator pass on labelled images, in the manner of
    tests/test_dcgan_discriminator.cu:49-136: layers, logits, loss, every dW / db, and the gradient of
    the images."""
    import __graft_entry__ as ge
    M = ge.load_package().hostabi.DcganModel
    names = [("disc_l%d" % i, "d_real_l%d" % i) for i in range(4)] + [("disc_logits", "d_real_logits"), ("disc_loss", "disc_loss")]
    names += [("grad_disc_loss_" + v, M.grad_name("disc_loss", v)) for v in D_VARS + ["x_real"]]
    return names


def collect_disc(model):
    """The tensors of disc_names() from ONE run of the graph (weights, images and labels already set)."""
    names = disc_names()
    got = model.eval_many([n for _, n in names])
    return {key: got[n] for key, n in names}


def torch_disc(w, x, y):
    """float64 torch evaluation of the labelled discriminator pass: same keys as collect_disc()."""
    import torch
    import torch.nn.functional as F
    T = {k: torch.tensor(w[k], dtype=torch.float64, requires_grad=True) for k in D_VARS}
    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    out, h = {}, xt
    for i in range(4):
        ht = F.pad(h.permute(0, 3, 1, 2), (1, 2, 1, 2))
        h = F.leaky_relu(F.conv2d(ht, T["d%d_w" % i].permute(3, 2, 0, 1), stride=2).permute(0, 2, 3, 1) + T["d%d_b" % i], 0.2)
        out["disc_l%d" % i] = h
    logits = h.reshape(x.shape[0], 8192) @ T["d4_w"] + T["d4_b"]
    out["disc_logits"] = logits
    out["disc_loss"] = F.binary_cross_entropy_with_logits(logits, torch.tensor(y, dtype=torch.float64))
    grads = torch.autograd.grad(out["disc_loss"], [T[v] for v in D_VARS] + [xt])
    res = {k: v.detach().numpy().reshape(-1) for k, v in out.items()}
    for v, g in zip(D_VARS + ["x_real"], grads):
        res["grad_disc_loss_" + v] = g.detach().numpy().reshape(-1)
    return res


def tensor_names():
    """(key in the dump, name the facade's dg_eval understands) of everything the parity tests compare."""
    import __graft_entry__ as ge
    M = ge.load_package().hostabi.DcganModel
    names = [("g_l%d" % i, "g_l%d" % i) for i in range(5)] + [("g_out", "g_out")]
    for br in ("d_fake", "d_real"):
        names += [("%s_l%d" % (br, i),) * 2 for i in range(4)] + [(br + "_logits",) * 2]
    names += [(n, n) for n in ("g_loss", "d_loss", "d_fake_loss", "d_real_loss")]
    names += [("grad_d_loss_" + v, M.grad_name("d_loss", v)) for v in D_VARS]
    names += [("grad_g_loss_" + v, M.grad_name("g_loss", v)) for v in G_VARS + ["x_fake"]]
    return names


def collect(model, steps=1, one_run=True):
    """Everything the parity test compares, from a DcganModel with weights and inputs set: every
    layer, loss and gradient on the unchanged parameters (one run of the graph for all of them, or
    one run per tensor), then `steps` iterations (D step, G step) and the parameters after them."""
    names = tensor_names()
    if one_run:
        got = model.eval_many([n for _, n in names])
        out = {key: got[n] for key, n in names}
    else:
        out = {key: model.eval(n) for key, n in names}
    losses = []
    for _ in range(steps):
        losses.append(model.d_step())
        losses.append(model.g_step())
    out["step_losses"] = np.array(losses, np.float32)
    for v in G_VARS + D_VARS:
        out["after_" + v] = model.var(v).reshape(-1)
    return out


def torch_dcgan(w, z, x):
    """float64 torch evaluation: returns (tensors, grads) with the same keys as collect()."""
    import torch
    import torch.nn.functional as F
    T = {k: torch.tensor(v, dtype=torch.float64, requires_grad=True) for k, v in w.items()}
    zt = torch.tensor(z, dtype=torch.float64)
    xt = torch.tensor(x, dtype=torch.float64)
    B = z.shape[0]

    def conv_t(h, k, b):  # h NHWC, k [kh,kw,Cout,Cin] -> SAME, stride 2, out = 2 * in
        full = F.conv_transpose2d(h.permute(0, 3, 1, 2), k.permute(3, 2, 0, 1), stride=2)
        Ho = h.shape[1] * 2
        return full[:, :, 1:1 + Ho, 1:1 + Ho].permute(0, 2, 3, 1) + b

    def conv(h, k, b):    # SAME, stride 2: pad (1, 2)
        ht = F.pad(h.permute(0, 3, 1, 2), (1, 2, 1, 2))
        return F.conv2d(ht, k.permute(3, 2, 0, 1), stride=2).permute(0, 2, 3, 1) + b

    out = {}
    h = torch.relu(zt @ T["g0_w"] + T["g0_b"]).reshape(B, 4, 4, 512)
    out["g_l0"] = h
    for i in (1, 2, 3):
        h = torch.relu(conv_t(h, T["g%d_w" % i], T["g%d_b" % i]))
        out["g_l%d" % i] = h
    h = conv_t(h, T["g4_w"], T["g4_b"])
    out["g_l4"] = h
    g_out = torch.tanh(h)
    g_out.retain_grad()
    out["g_out"] = g_out

    def disc(img, tag):
        h = img
        for i in range(4):
            h = F.leaky_relu(conv(h, T["d%d_w" % i], T["d%d_b" % i]), 0.2)
            out["%s_l%d" % (tag, i)] = h
        logits = h.reshape(B, 8192) @ T["d4_w"] + T["d4_b"]
        out[tag + "_logits"] = logits
        return logits

    fake, real = disc(g_out, "d_fake"), disc(xt, "d_real")
    ones, zeros = torch.ones_like(fake), torch.zeros_like(fake)
    bce = F.binary_cross_entropy_with_logits
    out["g_loss"] = bce(fake, ones)
    out["d_fake_loss"] = bce(fake, zeros)
    out["d_real_loss"] = bce(real, ones)
    out["d_loss"] = out["d_fake_loss"] + out["d_real_loss"]
    grads = {}
    gd = torch.autograd.grad(out["d_loss"], [T[v] for v in D_VARS], retain_graph=True)
    for v, g in zip(D_VARS, gd):
        grads["grad_d_loss_" + v] = g
    gg = torch.autograd.grad(out["g_loss"], [T[v] for v in G_VARS] + [g_out], retain_graph=True)
    for v, g in zip(G_VARS + ["x_fake"], gg):
        grads["grad_g_loss_" + v] = g
    res = {k: v.detach().numpy().reshape(-1) for k, v in out.items()}
    res.update({k: v.detach().numpy().reshape(-1) for k, v in grads.items()})
    return res


def main():
    batch, seed, path = int(sys.argv[1]), int(sys.argv[2]), sys.argv[3]
    disc = len(sys.argv) > 4 and sys.argv[4] == "disc"
    steps = int(sys.argv[4]) if len(sys.argv) > 4 and not disc else 1
    import __graft_entry__ as ge
    pkg = ge.load_package()
    f64 = len(sys.argv) > 5 and sys.argv[5] == "f64"
    backend = os.path.join(ROOT, "oracle", "liboracle_backend_f64.so" if f64 else "liboracle_backend.so")
    model = pkg.hostabi.DcganModel(batch, seed, "CPU", backend)
    w, z, x = synthetic(batch, seed, pkg.hostabi.var_shapes())
    for name, val in w.items():
        model.set_var(name, val)
    model.set_inputs(z, x)
    if disc:
        model.set_labels(labels(batch, seed))
        np.savez(path, **collect_disc(model))
    else:
        np.savez(path, **collect(model, steps))
    model.close()


if __name__ == "__main__":
    main()

#!/usr/bin/env python3
"""Write tests/golden/ref_literals.json: the literal inputs of the reference's own operator
tests plus expected outputs.

The reference's tests hold INPUTS only; their expected outputs came from TensorFlow 1.7 at test
time and were never stored.  This script therefore

  * reads the literal input arrays out of the reference's test sources as TEXT (C initialiser
    lists with a regex, numpy literals with ``ast`` -- nothing from the reference is imported
    or executed), and
  * computes the expected outputs in float64 by routes that are independent of the oracle:
    ``torch.nn.functional.conv2d`` / ``conv_transpose2d`` and torch autograd for the
    convolutions, numpy closed forms for everything else.

Three expected vectors (conv2d, conv2d_padding, conv2d_transpose) are additionally asserted against
integer values for the same inputs that were known before this script existed (the literal lists below).

Run once in a container that has the reference mounted:  python tests/golden/make_golden.py
The JSON it writes is committed; the tests never need the reference tree.
"""
import ast
import json
import os
import re
import sys

import numpy as np
import torch
import torch.nn.functional as F

REF = os.environ.get("DCGAN_REFERENCE", "/root/reference")
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_literals.json")


def c_arrays(path):
    """All `dbl_t name[...] = { ... };` initialiser lists of a C++ source, as float64 arrays."""
    text = open(os.path.join(REF, path)).read()
    text = re.sub(r"//[^\n]*", "", text)
    res = {}
    for m in re.finditer(r"dbl_t\s+(\w+)\s*\[\s*\d*\s*\]\s*=\s*\{([^}]*)\}", text):
        vals = [float(v.replace(" ", "")) for v in m.group(2).replace("\n", " ").split(",") if v.strip()]
        res[m.group(1)] = np.array(vals, dtype=np.float64)
    return res


def py_arrays(path):
    """All `name = np.array(<literal>)` assignments of a Python source (parsed, not run)."""
    tree = ast.parse(open(os.path.join(REF, path)).read())
    res = {}
    for node in tree.body:
        if isinstance(node, ast.Assign) and isinstance(node.value, ast.Call) \
                and getattr(node.value.func, "attr", "") == "array":
            res[node.targets[0].id] = np.array(ast.literal_eval(node.value.args[0]), dtype=np.float64)
    return res


def same_pads(n_in, k, s):
    p = max(k - s, 0) if n_in % s == 0 else max(k - n_in % s, 0)
    return p // 2, p - p // 2, p


def t_conv2d(x, k, s):
    """TF-SAME conv2d, NHWC x HWIO, float64, through torch."""
    N, H, W, C = x.shape
    kh, kw, _, O = k.shape
    pt, pb, _ = same_pads(H, kh, s)
    pl, pr, _ = same_pads(W, kw, s)
    xt = F.pad(x.permute(0, 3, 1, 2), (pl, pr, pt, pb))
    return F.conv2d(xt, k.permute(3, 2, 0, 1), stride=s).permute(0, 2, 3, 1)


def t_conv2d_transpose(x, k, out_hw, s):
    """TF conv2d_transpose with caller-supplied output size; k is [kh,kw,Cout,Cin]."""
    N, Hi, Wi, Ci = x.shape
    kh, kw, Co, _ = k.shape
    full = F.conv_transpose2d(x.permute(0, 3, 1, 2), k.permute(3, 2, 0, 1), stride=s)
    pad_h = (Hi - 1) * s + kh - out_hw[0]
    pad_w = (Wi - 1) * s + kw - out_hw[1]
    pt, pl = pad_h // 2, pad_w // 2
    return full[:, :, pt:pt + out_hw[0], pl:pl + out_hw[1]].permute(0, 2, 3, 1)


def T(a, shape, grad=False):
    t = torch.tensor(np.asarray(a, dtype=np.float64).reshape(shape))
    t.requires_grad_(grad)
    return t


def arr(a):
    a = np.asarray(a.detach().numpy() if isinstance(a, torch.Tensor) else a, dtype=np.float64)
    return {"shape": list(a.shape), "data": [float(v) for v in a.reshape(-1)]}


cases = []


def case(name, source, op, params, inputs, expected):
    cases.append({"name": name, "source": source, "op": op, "params": params,
                  "inputs": {k: arr(v) for k, v in inputs.items()},
                  "expected": {k: arr(v) for k, v in expected.items()}})


# ---- conv2d forward ------------------------------------------------------------------------
a = c_arrays("tests/test_conv2d.cu")
x, k = T(a["input"], (2, 4, 4, 2)), T(a["kernel"], (2, 2, 2, 2))
y = t_conv2d(x, k, 2)
assert y.reshape(-1).tolist() == [10, -6, 4, -1, -6, -14, 0, 2, 7, -6, 4, -11, 3, 5, 7, -9]
case("conv2d", "tests/test_conv2d.cu:28-50", "conv2d", {"strides": [2, 2]},
     {"x": x, "k": k}, {"y": y})

a = c_arrays("tests/test_conv2d_padding.cu")
x, k = T(a["input"], (2, 3, 5, 3)), T(a["kernel"], (2, 3, 3, 2))
y = t_conv2d(x, k, 2)
assert y.reshape(-1).tolist() == [2, 1, -10, 0, 10, -15, 3, 1, -8, -7, 15, -5, -13, 1, -10, 2,
                                  33, -4, 20, 7, -21, 1, 8, -8]
case("conv2d_padding", "tests/test_conv2d_padding.cu:28-78", "conv2d", {"strides": [2, 2]},
     {"x": x, "k": k}, {"y": y})


# ---- conv2d gradients through reshape -> mse -------------------------------------------------
def conv_grad_case(name, src, xs, ks, ys):
    a = c_arrays(src.split(":")[0])
    x, k = T(a["input"], xs, True), T(a["kernel"], ks, True)
    yt = T(a["y"], ys)
    y_hat = t_conv2d(x, k, 2)
    y_hat.retain_grad()
    loss = ((yt - y_hat) ** 2).mean()
    loss.backward()
    case(name, src, "conv2d_grad", {"strides": [2, 2]},
         {"x": x, "k": k, "y": yt},
         {"y_hat": y_hat, "dy_hat": y_hat.grad, "dx": x.grad, "dk": k.grad, "loss": loss})


conv_grad_case("conv2d_grad", "tests/test_conv2d_grad.cu:30-83", (2, 4, 4, 3), (2, 2, 3, 2), (2, 2, 2, 2))
conv_grad_case("conv2d_padding_grad", "tests/test_conv2d_padding_grad.cu:29-95",
               (2, 3, 5, 3), (2, 3, 3, 2), (2, 2, 3, 2))

# ---- conv2d_transpose ----------------------------------------------------------------------
a = c_arrays("tests/test_conv2d_transpose.cu")
x, k = T(a["input"], (2, 2, 2, 1)), T(a["kernel"], (2, 2, 1, 1))
y = t_conv2d_transpose(x, k, (4, 4), 2)
assert y.reshape(-1).tolist() == [
    -0.125, 0.125, -2.25, 2.25, 0.125, -0.125, 2.25, -2.25, -1.75, 1.75, -0.25, 0.25, 1.75, -1.75,
    0.25, -0.25, -0.5, 0.5, 3, -3, 0.5, -0.5, -3, 3, 0.25, -0.25, -0.375, 0.375, -0.25, 0.25,
    0.375, -0.375]
case("conv2d_transpose", "tests/test_conv2d_transpose.cu:28-45", "conv2d_transpose",
     {"strides": [2, 2], "out_size": [2, 4, 4, 1]}, {"x": x, "k": k}, {"y": y})

a = c_arrays("tests/test_conv2d_transpose_grad.cu")
x, k = T(a["input"], (2, 4, 4, 3), True), T(a["kernel"], (2, 2, 2, 3), True)
yt = T(a["y"], (2, 8, 8, 2))
y_hat = t_conv2d_transpose(x, k, (8, 8), 2)
y_hat.retain_grad()
loss = ((yt - y_hat) ** 2).mean()
loss.backward()
case("conv2d_transpose_grad", "tests/test_conv2d_transpose_grad.cu:30-233", "conv2d_transpose_grad",
     {"strides": [2, 2], "out_size": [2, 8, 8, 2]}, {"x": x, "k": k, "y": yt},
     {"y_hat": y_hat, "dy_hat": y_hat.grad, "dx": x.grad, "dk": k.grad, "loss": loss})

# ---- bias add and its gradient -----------------------------------------------------------------
a = c_arrays("tests/test_conv2d_bias_add.cu")
z, b = a["input"].reshape(2, 2, 2, 2), a["bias"]
case("conv2d_bias_add", "tests/test_conv2d_bias_add.cu:28-34", "bias_add", {},
     {"z": z, "b": b}, {"out": z + b})

a = c_arrays("tests/test_conv2d_bias_add_grad.cu")
z, b, yt = a["input"].reshape(2, 2, 2, 2), a["bias"], a["y"].reshape(2, 2, 2, 2)
dy_hat = 2.0 / z.size * ((z + b) - yt)
case("conv2d_bias_add_grad", "tests/test_conv2d_bias_add_grad.cu:29-43", "bias_add_grad", {},
     {"z": z, "b": b, "y": yt},
     {"dy_hat": dy_hat, "dx": dy_hat, "db": dy_hat.reshape(-1, 2).sum(0)})

# ---- activations -------------------------------------------------------------------------------
a = py_arrays("tests/ref_vect_relu_leaky.py")["features"]
case("vect_relu_leaky", "tests/ref_vect_relu_leaky.py:10", "relu_leaky", {"alpha": 0.2},
     {"x": a}, {"out": np.where(a < 0, 0.2 * a, a)})
a = py_arrays("tests/ref_vect_relu.py")["features"]
case("vect_relu", "tests/ref_vect_relu.py:10", "relu", {}, {"x": a}, {"out": np.maximum(a, 0)})
a = py_arrays("tests/ref_vect_tanh.py")["features"]
case("vect_tanh", "tests/ref_vect_tanh.py:10", "tanh", {}, {"x": a}, {"out": np.tanh(a)})
a = py_arrays("tests/ref_sigmoid.py")["logits"]
case("sigmoid", "tests/ref_sigmoid.py:10-15", "sigmoid", {}, {"x": a}, {"out": 1 / (1 + np.exp(-a))})


def act_grad_case(name, src, fn, dfn_from, alpha=None):
    a = py_arrays(src.split(":")[0])
    x, yt = a["x"], a["y"]
    y_hat = fn(x)
    dy_hat = 2.0 / x.size * (y_hat - yt)
    dx = dfn_from(x, y_hat) * dy_hat
    p = {} if alpha is None else {"alpha": alpha}
    case(name, src, name, p, {"x": x, "y": yt}, {"y_hat": y_hat, "dy_hat": dy_hat, "dx": dx})


act_grad_case("leaky_relu_grad", "tests/ref_leaky_relu_grad.py:10-22",
              lambda x: np.where(x < 0, 0.3 * x, x), lambda x, o: np.where(x < 0, 0.3, 1.0), 0.3)
act_grad_case("relu_grad", "tests/ref_relu_grad.py:10-22",
              lambda x: np.maximum(x, 0), lambda x, o: (x > 0).astype(np.float64))
act_grad_case("tanh_grad", "tests/ref_tanh_grad.py:10-22", np.tanh, lambda x, o: 1 - o * o)
act_grad_case("sigmoid_grad", "tests/ref_sigmoid_grad.py:10-22",
              lambda x: 1 / (1 + np.exp(-x)), lambda x, o: o * (1 - o))

# ---- add, argmax, sigmoid cross-entropy --------------------------------------------------------
a = py_arrays("tests/ref_add.py")
case("add", "tests/ref_add.py:10-22", "add", {}, {"a": a["a"], "b": a["b"]}, {"out": a["a"] + a["b"]})

a = py_arrays("tests/ref_argmax.py")
acc = float((a["y"].argmax(1) == a["y_hat"].argmax(1)).sum())
case("argmax_accuracy", "tests/ref_argmax.py:10-35", "argmax_acc", {},
     {"y": a["y"], "y_hat": a["y_hat"]}, {"acc": np.array(acc)})

a = py_arrays("tests/ref_sigmoid_cross_entropy_grad.py")
x, yl = a["x"], a["y"]
ce = np.maximum(x, 0) - x * yl + np.log1p(np.exp(-np.abs(x)))
case("sigmoid_cross_entropy", "tests/ref_sigmoid_cross_entropy.py:10-24", "sigmoid_cross_entropy", {},
     {"x": x, "y": yl}, {"loss": np.array(ce.mean()), "dx": (1 / (1 + np.exp(-x)) - yl) / x.size})

# ---- Adam ----------------------------------------------------------------------------------------
a = py_arrays("tests/ref_moment_update.py")
case("moment_update", "tests/test_moment_update.cu:33-53", "moment_update", {"c1": 5.7, "c2": 3.9},
     {"var": a["a"], "dv": a["b"]}, {"out": 5.7 * a["a"] + 3.9 * a["b"]})
a = py_arrays("tests/ref_moment_update2.py")
case("moment_update2", "tests/ref_moment_update2.py:10-24", "moment_update2", {"c1": 5.7, "c2": 3.9},
     {"var": a["a"], "dv": a["b"]}, {"out": 5.7 * a["a"] + 3.9 * a["b"] * a["b"]})
a = py_arrays("tests/ref_adam_update.py")
lr, b1, b2, eps, t = 0.45, 0.68, 0.27, 2.0, 1
lrt = lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)
case("adam_update", "tests/test_adam_update.cu:33-56", "adam_update",
     {"lr": lr, "beta1": b1, "beta2": b2, "eps": eps, "t_before": 0},
     {"x": a["x"], "m": a["m"], "v": a["v"]},
     {"out": a["x"] - lrt * a["m"] / (np.sqrt(a["v"]) + eps)})

# ---- dense ---------------------------------------------------------------------------------------
a = py_arrays("tests/ref_mat_mul_add.py")
case("mat_mul_add", "tests/ref_mat_mul_add.py:10-24", "mat_mul_add", {},
     {"x": a["x"], "w": a["w"], "b": a["b"]}, {"out": a["x"] @ a["w"] + a["b"]})
a = py_arrays("tests/ref_mat_mat_mul.py")
case("mat_mat_mul", "tests/ref_mat_mat_mul.py:10-22", "mm_mul", {}, {"a": a["a"], "b": a["b"]},
     {"out": a["a"] @ a["b"]})
a = py_arrays("tests/ref_tmat_mat_mul.py")
case("tmat_mat_mul", "tests/ref_tmat_mat_mul.py:10-21", "tmm_mul", {}, {"a": a["a"], "b": a["b"]},
     {"out": a["a"].T @ a["b"]})
a = py_arrays("tests/ref_mat_tmat_mul.py")
case("mat_tmat_mul", "tests/ref_mat_tmat_mul.py:10-21", "mtm_mul", {}, {"a": a["a"], "b": a["b"]},
     {"out": a["a"] @ a["b"].T})
a = py_arrays("tests/ref_mat_rvect_add.py")
case("mat_rvect_add", "tests/ref_mat_rvect_add.py:10-19", "bias_add", {},
     {"z": a["a"], "b": a["b"].reshape(-1)}, {"out": a["a"] + a["b"]})
a = py_arrays("tests/ref_mat_sum0.py")
case("mat_sum_cols", "tests/ref_mat_sum0.py:10-14", "mat_sum_cols", {}, {"x": a["x"]},
     {"out": a["x"].sum(0)})

json.dump({"generator": "tests/golden/make_golden.py", "cases": cases}, open(OUT, "w"), indent=0)
print("wrote", OUT, len(cases), "cases", os.path.getsize(OUT), "bytes", file=sys.stderr)

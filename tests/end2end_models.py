"""The reference's End2End test models (test/End2End/{CPU,GPU}/*.mlir) as device
plans, with the constants those files embed (tests/golden/end2end_constants.npz,
written by tests/golden/make_end2end_fixtures.py).  Shared by the CPU-runner
and GPU-runner tests; expected outputs come from the oracle."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
MODELS = json.load(open(os.path.join(HERE, "golden", "end2end_models.json")))
CONSTANTS = dict(np.load(os.path.join(HERE, "golden", "end2end_constants.npz")))


def dims(shape):
    return "x".join(str(d) for d in shape) + "xf32"


def ints(v):
    return "[" + ", ".join(str(i) for i in v) + "]"


def build(name, directory, device):
    """Writes <directory>/<name>.plan and its constant files; returns
    (plan path, input shapes, output shape, reference function over the inputs)."""
    m = MODELS[name]
    x = dims(m["inputs"][0])
    y = dims(m["output"])
    consts = {}
    if name == "add":
        body = f"func @main_graph(%a: {x}, %b: {x}) -> (%c: {y}) {{\n  %c = device.add %a, %b : {y}\n  return\n}}\n"
        ref = lambda oracle, a, b: oracle.add_f32(a, b)
    elif name in ("add_constant", "add_constant_splat"):
        consts["addend"] = CONSTANTS[name]
        body = (f"func @main_graph(%a: {x}) -> (%c: {y}) {{\n  %k = device.constant {{file = \"addend.dat\"}} : {y}\n"
                f"  %c = device.add %a, %k : {y}\n  return\n}}\n")
        ref = lambda oracle, a: oracle.add_f32(a, CONSTANTS[name])
    elif name == "linear":
        w, b = CONSTANTS["linear_weight"], CONSTANTS["linear_bias"]
        consts["weight"], consts["bias"] = w, b
        head = (f"func @main_graph(%x: {x}) -> (%y: {y}) {{\n  %w = device.constant {{file = \"weight.dat\"}} : {dims(w.shape)}\n"
                f"  %b = device.constant {{file = \"bias.dat\"}} : {dims(b.shape)}\n")
        if device == "gpu":  # MatMul + Add + Relu as one call with the ReLU epilogue
            body = head + f"  %y = device.matmul-ex %x, %w, %b, none {{act = \"relu\"}} : {y}\n  return\n}}\n"
            ref = lambda oracle, a: np.maximum(a.astype(np.float64) @ w + b, 0.0)
        else:  # the CPU op library has the bias form only (ConvertDeviceToLLVM.cpp:433-436): pre-activation
            body = head + f"  %y = device.matmul %x, %w, %b : {y}\n  return\n}}\n"
            ref = lambda oracle, a: a.astype(np.float64) @ w + b
    elif name == "conv":
        w, b = CONSTANTS["conv_weight"], CONSTANTS["conv_bias"]
        consts["weight"], consts["bias"] = w, b
        body = (f"func @main_graph(%x: {x}) -> (%y: {y}) {{\n  %w = device.constant {{file = \"weight.dat\"}} : {dims(w.shape)}\n"
                f"  %b = device.constant {{file = \"bias.dat\"}} : {dims(b.shape)}\n"
                f"  %y = device.conv2d %x, %w, %b, none {{kernel = {ints(m['kernel'])}, pad = {ints(m['pad'])}, "
                f"stride = {ints(m['stride'])}, dilation = {ints(m['dilation'])}, containRelu = false}} : {y}\n  return\n}}\n")
        ref = lambda oracle, a: oracle.conv2d(a, w, b, None, tuple(m["pad"]), tuple(m["stride"]), tuple(m["dilation"]), False)
    elif name == "pool":
        body = (f"func @main_graph(%x: {x}) -> (%y: {y}) {{\n  %y = device.pool2d %x {{kernel = {ints(m['kernel'])}, "
                f"pad = {ints(m['pad'])}, stride = {ints(m['stride'])}, method = \"{m['method']}\"}} : {y}\n  return\n}}\n")
        ref = lambda oracle, a: oracle.pool2d(a, tuple(m["kernel"]), tuple(m["pad"]), tuple(m["stride"]), m["method"])
    else:
        raise KeyError(name)
    os.makedirs(directory, exist_ok=True)
    for cname, arr in consts.items():
        np.ascontiguousarray(arr, np.float32).tofile(os.path.join(directory, cname + ".dat"))
    plan = os.path.join(directory, name + ".plan")
    with open(plan, "w") as f:
        f.write(body)
    return plan, m["inputs"], m["output"], ref

#!/usr/bin/env python3
"""Writes tests/golden/end2end_constants.npz and tests/golden/end2end_models.json.

The reference's End2End tests (test/End2End/{CPU,GPU}/{add,linear,conv,pool}.mlir;
the CPU and GPU copies differ only in their RUN line) are ONNX-dialect modules
with the model constants embedded: a (2,10,10) addend, a 32x64 linear weight
and its bias, a 64x3x3x3 filter and its bias.  They hold inputs only - the lit
RUN line checks that the pipeline exits 0 - so these fixtures carry the
constants (data, as dense<"0x..."> hex, dense<[...]> lists or splats) and the
operator attributes, nothing else; expected outputs come from the oracle in
the tests.  Only possible where the reference checkout is present.

    python tests/golden/make_end2end_fixtures.py
"""
import json
import os
import re

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/test/End2End/GPU"


def shape_of(tensor_type):
    dims = tensor_type.split("x")
    assert dims[-1] == "f32", tensor_type
    return [int(d) for d in dims[:-1]]


def constants(text):
    """[(array, shape)] for every onnx.Constant of a module, in order."""
    out = []
    for m in re.finditer(r'onnx\.Constant dense<(.*?)>\s*:\s*tensor<([0-9x]*f32)>', text, re.S):
        body, shape = m.group(1).strip(), shape_of(m.group(2))
        n = int(np.prod(shape))
        if body.startswith('"0x'):
            a = np.frombuffer(bytes.fromhex(body[3:-1]), dtype="<f4")
        elif body.startswith("["):
            a = np.array([float(v) for v in body.strip("[]").split(",")], np.float32)
        else:  # splat
            a = np.full(n, float(body), np.float32)
        assert a.size == n, (a.size, shape)
        out.append(a.reshape(shape).astype(np.float32))
    return out


def int_list(text, key):
    m = re.search(key + r"\s*=\s*\[([0-9, ]*)\]", text)
    return [int(v) for v in m.group(1).split(",")] if m else None


def main():
    arrays, models = {}, {}
    read = lambda name: open(os.path.join(REF, name)).read()

    mods = read("add.mlir").split("// -----")
    assert len(mods) == 3
    models["add"] = {"inputs": [[3, 640, 640], [3, 640, 640]], "output": [3, 640, 640]}
    (c1,), (c2,) = constants(mods[1]), constants(mods[2])
    arrays["add_constant"] = c1
    arrays["add_constant_splat"] = c2
    models["add_constant"] = {"inputs": [list(c1.shape)], "output": list(c1.shape)}
    models["add_constant_splat"] = {"inputs": [list(c2.shape)], "output": list(c2.shape)}

    text = read("linear.mlir")
    bias, weight = constants(text)  # the bias constant comes first in the file
    assert weight.ndim == 2 and bias.shape == (weight.shape[1],)
    assert re.findall(r'"onnx\.(MatMul|Add|Relu)"', text) == ["MatMul", "Add", "Relu"]
    arrays["linear_weight"], arrays["linear_bias"] = weight, bias
    models["linear"] = {"inputs": [[3, 32, weight.shape[0]]], "output": [3, 32, weight.shape[1]], "relu": True}

    text = read("conv.mlir")
    weight, bias = constants(text)
    assert weight.ndim == 4 and bias.shape == (weight.shape[0],)
    pads = int_list(text, "pads")  # ONNX order: top, left, bottom, right
    models["conv"] = {"inputs": [[16, 3, 256, 256]], "output": [16, weight.shape[0], 256, 256],
                      "kernel": int_list(text, "kernel_shape"), "pad": pads, "stride": int_list(text, "strides"),
                      "dilation": int_list(text, "dilations")}
    arrays["conv_weight"], arrays["conv_bias"] = weight, bias

    text = read("pool.mlir")
    models["pool"] = {"inputs": [[16, 3, 256, 256]], "output": [16, 3, 64, 64], "kernel": int_list(text, "kernel_shape"),
                      "pad": int_list(text, "pads"), "stride": int_list(text, "strides"), "method": "max"}

    np.savez_compressed(os.path.join(HERE, "end2end_constants.npz"), **arrays)
    with open(os.path.join(HERE, "end2end_models.json"), "w") as f:
        json.dump(models, f, indent=1, sort_keys=True)
        f.write("\n")
    for k, v in arrays.items():
        print(k, v.shape, float(np.abs(v).max()))


if __name__ == "__main__":
    main()

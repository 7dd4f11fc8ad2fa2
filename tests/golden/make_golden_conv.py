"""Writes ``conv_cases.npz`` by RUNNING THE REFERENCE's convolution layers on the CPU.

Run once, in the build container, where the reference is mounted read-only:

    PYTHONPATH=/root/reference/src python tests/golden/make_golden_conv.py

Evaluates ``CONV_CASES`` (torch-mode, CPU, fixed seeds) with the reference's ``AnalogConv1d``,
``AnalogConv2d`` and ``AnalogConv3d`` and stores outputs and gradients (bf16 as float32, which
holds it exactly). Only data is written. The fixtures pin the patch order against the weight
view, the tile split of the patch dimension, the output layout and the fold of the gradient.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from conv_cases import CONV_CASES, make_conv_inputs  # noqa: E402  pylint: disable=wrong-import-position
from golden_cases import DTYPES  # noqa: E402  pylint: disable=wrong-import-position
from make_golden import f32, ref_config  # noqa: E402  pylint: disable=wrong-import-position

from aihwkit_lightning.nn import AnalogConv1d, AnalogConv2d, AnalogConv3d  # noqa: E402  (the reference)

LAYERS = {1: AnalogConv1d, 2: AnalogConv2d, 3: AnalogConv3d}


def run_case(case, store):
    name, dtype = case["name"], DTYPES[case["dtype"]]
    x, w, b, g = make_conv_inputs(case)
    one = case["ndim"] == 1
    layer = LAYERS[case["ndim"]](
        case["C"], case["N"],
        case["kernel"][0] if one else case["kernel"],
        stride=case["stride"][0] if one else case["stride"],
        padding=case["padding"][0] if one else case["padding"],
        dilation=case["dilation"][0] if one else case["dilation"],
        bias=b is not None, dtype=dtype, rpu_config=ref_config(case),
    )
    layer.set_weights_and_biases(w.unsqueeze(-2) if one else w, b)
    if case["ir_values"] is not None and layer.input_range is not None:
        layer.input_range.data = torch.tensor(case["ir_values"], dtype=dtype)
    layer.train(case["training"])
    xin = x.clone().requires_grad_(True)
    torch.manual_seed(case["noise_seed"])
    out = layer(xin)
    out.backward(g)
    store[f"{name}/out"] = f32(out)
    store[f"{name}/dx"] = f32(xin.grad)
    wgrad = layer.weight.grad
    store[f"{name}/dw"] = f32(wgrad.squeeze(-2) if one else wgrad)
    if b is not None:
        store[f"{name}/db"] = f32(layer.bias.grad)
    if layer.input_range is not None and layer.input_range.grad is not None:
        store[f"{name}/dir"] = f32(layer.input_range.grad)


def main():
    store = {}
    for case in CONV_CASES:
        run_case(case, store)
        print("done", case["name"])
    path = os.path.join(HERE, "conv_cases.npz")
    np.savez_compressed(path, **store)
    print(f"wrote {path}: {os.path.getsize(path) / 1e3:.1f} kB, {len(store)} arrays")


if __name__ == "__main__":
    main()

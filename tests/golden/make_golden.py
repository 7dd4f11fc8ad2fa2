"""Writes the golden fixtures of this directory by RUNNING THE REFERENCE on the CPU.

Run once, in the build container, where the reference is mounted read-only:

    PYTHONPATH=/root/reference/src python tests/golden/make_golden.py

It imports ``aihwkit_lightning`` from the reference (torch-mode, CPU), evaluates the cases in
``CASES`` with fixed seeds and stores inputs and outputs in ``linear_cases.npz`` (bf16 tensors are
stored as float32, which holds them exactly). Only data is written; nothing of the reference's
code travels. The fixtures pin what no closed form pins: the composite forward (op order and the
sequence of dtype roundings), the input-range gradient with its decay switch, weight gradients
under clamp masks and weight noise, the input-range initialisation sequence.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, HERE)
from golden_cases import CASES, DTYPES, make_inputs, make_learnable_clip  # noqa: E402  pylint: disable=wrong-import-position

from aihwkit_lightning.nn import AnalogLinear  # noqa: E402  (the reference)
from aihwkit_lightning.optim import AnalogOptimizer  # noqa: E402
from aihwkit_lightning.simulator.configs import (  # noqa: E402
    TorchInferenceRPUConfig,
    WeightClipType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
)

CLIP = {
    "none": WeightClipType.NONE,
    "layer": WeightClipType.LAYER_GAUSSIAN,
    "channel": WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL,
    "learnable": WeightClipType.LEARNABLE_PER_CHANNEL,
}
QUANT = {
    "none": WeightQuantizationType.NONE,
    "discretize": WeightQuantizationType.DISCRETIZE,
    "discretize_per_channel": WeightQuantizationType.DISCRETIZE_PER_CHANNEL,
}
NOISE = {
    "none": WeightNoiseInjectionType.NONE,
    "add_normal": WeightNoiseInjectionType.ADD_NORMAL,
    "add_normal_per_channel": WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL,
}


def ref_config(case) -> TorchInferenceRPUConfig:
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = case["max_input_size"]
    cfg.forward.inp_res = case["inp_res"]
    cfg.forward.out_res = case["out_res"]
    cfg.forward.out_bound = case["out_bound"]
    cfg.forward.out_noise = case["out_noise"]
    cfg.forward.out_noise_per_channel = case["out_noise_per_channel"]
    cfg.clip.type = CLIP[case["clip"]]
    cfg.clip.sigma = case["clip_sigma"]
    cfg.modifier.quantization_type = QUANT[case["weight_quant"]]
    cfg.modifier.noise_type = NOISE[case["weight_noise"]]
    cfg.modifier.res = case["modifier_res"]
    cfg.modifier.std_dev = case["modifier_std"]
    ir = cfg.pre_post.input_range
    ir.enable = case["ir_mode"] != "none"
    ir.dynamic = case["ir_mode"] == "dynamic"
    ir.fast_mode = case["ir_mode"] == "fast"
    ir.act_range_momentum = case["act_range_momentum"]
    ir.init_value = case["ir_init"]
    ir.init_from_data = case["init_from_data"]
    ir.init_std_alpha = case["init_std_alpha"]
    ir.decay = case["ir_decay"]
    ir.input_min_percentage = case["ir_min_pct"]
    return cfg


def f32(t):
    return None if t is None else t.detach().float().numpy()


def run_case(case, store):
    name, dtype = case["name"], DTYPES[case["dtype"]]
    x, w, b, g = make_inputs(case)
    layer = AnalogLinear(case["K"], case["N"], bias=b is not None, dtype=dtype,
                         rpu_config=ref_config(case))
    layer.set_weights_and_biases(w, b)
    if case["ir_values"] is not None and layer.input_range is not None:
        layer.input_range.data = torch.tensor(case["ir_values"], dtype=dtype)
    if case["clip"] == "learnable":
        layer.learnable_weight_clip.data = make_learnable_clip(case, w)
    layer.train(case["training"])
    kind = case["kind"]
    if kind == "fwd_bwd":
        xin = x.clone().requires_grad_(True)
        torch.manual_seed(case["noise_seed"])
        out = layer(xin)
        out.backward(g)
        store[f"{name}/out"] = f32(out)
        store[f"{name}/dx"] = f32(xin.grad)
        store[f"{name}/dw"] = f32(layer.weight.grad)
        if b is not None:
            store[f"{name}/db"] = f32(layer.bias.grad)
        if layer.input_range is not None and layer.input_range.grad is not None:
            store[f"{name}/dir"] = f32(layer.input_range.grad)
        if case["clip"] == "learnable":
            store[f"{name}/dlwc"] = f32(layer.learnable_weight_clip.grad)
    elif kind == "ir_init":
        for step in range(case["steps"]):
            torch.manual_seed(case["noise_seed"] + step)
            xs = torch.randn_like(x) * (1.0 + step)
            out = layer(xs)
            store[f"{name}/x{step}"] = f32(xs)
            store[f"{name}/out{step}"] = f32(out)
            store[f"{name}/ir{step}"] = f32(layer.input_range.data.clone())
            store[f"{name}/idx{step}"] = f32(layer.input_range_update_idx.clone())
    elif kind == "ir_fast_init":
        for step in range(case["steps"]):
            torch.manual_seed(case["noise_seed"] + step)
            xs = torch.randn_like(x) * (1.0 + step) + 0.25 * step
            out = layer(xs)
            store[f"{name}/x{step}"] = f32(xs)
            store[f"{name}/out{step}"] = f32(out)
            store[f"{name}/ir{step}"] = f32(layer.input_range.data.clone())
            store[f"{name}/idx{step}"] = f32(layer.input_range_update_idx.clone())
            store[f"{name}/xmin{step}"] = f32(layer.x_min.clone())
            store[f"{name}/xmax{step}"] = f32(layer.x_max.clone())
    elif kind == "clip":
        optim = AnalogOptimizer(torch.optim.SGD, layer.analog_layers, layer.parameters(), lr=0.0)
        layer(x).sum().backward()
        optim.step()
        store[f"{name}/w_clipped"] = f32(layer.weight.data)
    elif kind == "quantize":
        import warnings
        with warnings.catch_warnings():
            warnings.simplefilter("ignore")
            layer.quantize_weights()
        store[f"{name}/w_quantized"] = f32(layer.weight.data)
        layer.eval()
        store[f"{name}/out"] = f32(layer(x))
    else:
        raise ValueError(kind)


def main():
    store = {}
    for case in CASES:
        run_case(case, store)
        print("done", case["name"])
    path = os.path.join(HERE, "linear_cases.npz")
    np.savez_compressed(path, **store)
    print(f"wrote {path}: {os.path.getsize(path) / 1e6:.2f} MB, {len(store)} arrays")


if __name__ == "__main__":
    main()

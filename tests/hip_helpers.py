"""Helpers of the GPU parity tests: build the product layer for a case, run it, fetch results."""
import torch

from golden_cases import DTYPES, make_inputs, make_learnable_clip
from helpers import case_input_range

from aihwkit_lightning.nn import AnalogLinear
from aihwkit_lightning.simulator.configs import (
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


def rpu_config(c) -> TorchInferenceRPUConfig:
    """The package's RPU config of a case dict (same fields as tests/golden/golden_cases.py)."""
    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = c["max_input_size"]
    cfg.forward.inp_res = c["inp_res"]
    cfg.forward.out_res = c["out_res"]
    cfg.forward.out_bound = c["out_bound"]
    cfg.forward.out_noise = c["out_noise"]
    cfg.forward.out_noise_per_channel = c["out_noise_per_channel"]
    cfg.clip.type = CLIP[c["clip"]]
    cfg.clip.sigma = c["clip_sigma"]
    cfg.modifier.quantization_type = QUANT[c["weight_quant"]]
    cfg.modifier.noise_type = NOISE[c["weight_noise"]]
    cfg.modifier.res = c["modifier_res"]
    cfg.modifier.std_dev = c["modifier_std"]
    ir = cfg.pre_post.input_range
    ir.enable = c["ir_mode"] != "none"
    ir.dynamic = c["ir_mode"] == "dynamic"
    ir.fast_mode = c["ir_mode"] == "fast"
    ir.act_range_momentum = c["act_range_momentum"]
    ir.init_value = c["ir_init"]
    ir.init_from_data = c["init_from_data"]
    ir.init_std_alpha = c["init_std_alpha"]
    ir.decay = c["ir_decay"]
    ir.input_min_percentage = c["ir_min_pct"]
    return cfg


def make_layer(c, device="cuda", inputs=None):
    """AnalogLinear on the device with the case's weights, bias and input ranges."""
    dtype = DTYPES[c["dtype"]]
    _, w, b, _ = inputs if inputs is not None else make_inputs(c)
    layer = AnalogLinear(c["K"], c["N"], bias=b is not None, dtype=dtype, rpu_config=rpu_config(c))
    layer.set_weights_and_biases(w, b)
    layer = layer.to(device)
    if c["clip"] == "learnable":
        layer.learnable_weight_clip.data = make_learnable_clip(c, w).to(device)
    ir = case_input_range(c, len(layer.in_sizes))
    if ir is not None:
        layer.input_range.data = ir.to(device)
    layer.train(c["training"])
    return layer


def hip_fwd_bwd(c, inputs=None):
    """Forward + backward of the product layer; results on the CPU."""
    x, w, b, g = inputs if inputs is not None else make_inputs(c)
    layer = make_layer(c, inputs=(x, w, b, g))
    xin = x.cuda().requires_grad_(True)
    torch.manual_seed(c["noise_seed"])
    out = layer(xin)
    out.backward(g.cuda())
    torch.cuda.synchronize()
    res = dict(out=out.detach().cpu(), dx=xin.grad.cpu(), dw=layer.weight.grad.cpu(), db=None, dir=None)
    if b is not None:
        res["db"] = layer.bias.grad.cpu()
    if layer.input_range is not None and layer.input_range.grad is not None:
        res["dir"] = layer.input_range.grad.cpu()
    if layer.learnable_weight_clip is not None and layer.learnable_weight_clip.grad is not None:
        res["dlwc"] = layer.learnable_weight_clip.grad.cpu()
    return res

"""The binding a maintainer of the reference would write, tested: a ``torch.autograd.Function``
with the argument list of the reference's accelerated-operator slot
(``TritonLinear.apply(inp, weights, input_range, input_range_update_idx, learnable_weight_clip,
upper_end_of_slices, rpu_config, training)``, reference ``nn/modules/linear.py:125-134``,
``triton_utils/triton_linear.py:446-456``) on top of ``libanalog_hip.so`` with nothing but ctypes
and torch tensors for memory: its own mirror of the two configuration structs, no import from
this repository's host layer inside the function. Checked against this repository's
``AnalogLinear`` (which goes through the same library and is itself held to the oracle and the
reference's golden vectors by the other GPU tests) bit for bit with the noise off.

The function covers what the slot covers once the ranges are set: static learned range or
dynamic range or none, DAC / ADC / clamp, output noise and additive weight noise in training,
the straight-through backward with the clamp mask, the input-range gradient. Like the
reference's slot it returns the output without bias.
"""
import ctypes
import os
from ctypes import POINTER, byref, c_float, c_int32, c_int64, c_uint32, c_uint64, c_void_p

import pytest
import torch

pytestmark = pytest.mark.gpu

AHL_IR_NONE, AHL_IR_STATIC, AHL_IR_DYNAMIC = 0, 1, 2
AHL_DTYPE = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
AHL_NOISE_NONE, AHL_NOISE_ADD_NORMAL, AHL_NOISE_ADD_NORMAL_PER_CHANNEL = 0, 1, 2


class AhlLinearCfg(ctypes.Structure):          # struct AhlLinearCfg of include/analog_hip.h
    _fields_ = [("dtype", c_int32), ("ir_mode", c_int32), ("inp_res", c_float),
                ("out_res", c_float), ("out_bound", c_float), ("out_noise", c_float),
                ("out_noise_per_channel", c_int32), ("bound_per_channel", c_int32),
                ("training", c_int32), ("skip_rounding", c_int32), ("ir_decay", c_float),
                ("ir_input_min_percentage", c_float), ("ir_grad_rule", c_int32),
                ("tile_stride", c_int32), ("flag_token", c_uint32), ("seed", c_uint64),
                ("offset", c_uint64), ("seed_state", c_void_p)]


class AhlModifierCfg(ctypes.Structure):        # struct AhlModifierCfg
    _fields_ = [("dtype", c_int32), ("quant_type", c_int32), ("noise_type", c_int32),
                ("res", c_float), ("std_dev", c_float), ("wmax_given", c_int32),
                ("skip_tile_stats", c_int32), ("seed", c_uint64), ("offset", c_uint64),
                ("seed_state", c_void_p)]


def _load():
    import aihwkit_lightning  # only to find the built library next to the package

    path = os.path.join(os.path.dirname(aihwkit_lightning.__file__), "_lib", "libanalog_hip.so")
    lib = ctypes.CDLL(path)
    vp, i64, i32 = c_void_p, c_int64, c_int32
    ends, lcfg, mcfg = POINTER(c_int32), POINTER(AhlLinearCfg), POINTER(AhlModifierCfg)
    lib.ahl_weight_prep.argtypes = [vp, i64, i64, i64, ends, i32, mcfg, vp, vp, vp, vp, i64, vp]
    lib.ahl_dac.argtypes = [vp, i64, vp, i64, vp, vp, i64, i64, ends, i32, lcfg, vp]
    lib.ahl_linear_fwd.argtypes = [vp, i64, vp, i64, vp, i64, vp, vp, i64, vp, vp, vp, vp, vp,
                                   i64, i64, i64, ends, i32, lcfg, vp, vp]
    lib.ahl_linear_bwd_dx.argtypes = [vp, i64, vp, vp, vp, i64, vp, i64, vp, vp, i64, vp,
                                      i64, i64, i64, ends, i32, lcfg, vp, vp]
    lib.ahl_linear_bwd_dw.argtypes = [vp, i64, vp, vp, vp, i64, vp, i64, vp, vp, i64, vp,
                                      i64, i64, i64, ends, i32, lcfg, vp, vp]
    lib.ahl_linear_bwd_dx_ws_bytes.restype = c_int64
    lib.ahl_linear_bwd_dx_ws_bytes.argtypes = [i64, i64, i64, i32, i32, i64]
    lib.ahl_linear_bwd_dw_ws_bytes.restype = c_int64
    lib.ahl_linear_bwd_dw_ws_bytes.argtypes = [i64, i64, i64, i32, i32, i32, i64]
    return lib


def _p(tensor):
    return None if tensor is None else c_void_p(tensor.data_ptr())


def _ok(status, what):
    if status != 0:
        raise RuntimeError(f"{what} failed with status {status}")


class HipSlotLinear(torch.autograd.Function):
    """The reference's operator slot on libanalog_hip.so."""

    LIB = None

    @staticmethod
    def forward(ctx, inp, weights, input_range, input_range_update_idx, learnable_weight_clip,
                upper_end_of_slices, rpu_config, training):
        # pylint: disable=arguments-differ, unused-argument
        lib = HipSlotLinear.LIB
        assert learnable_weight_clip is None, "bind ahl_weight_prep with wmax_given for the learned clip"
        fwd, mod, irp = rpu_config.forward, rpu_config.modifier, rpu_config.pre_post.input_range
        x = inp.reshape(-1, inp.size(-1)).contiguous()
        w = weights.contiguous()
        m_rows, k_in = x.shape
        n_out = w.size(0)
        n_tiles = upper_end_of_slices.numel()
        ends = (c_int32 * n_tiles)(*[int(e) for e in upper_end_of_slices.tolist()])
        stream = c_void_p(torch.cuda.current_stream().cuda_stream)
        dt = AHL_DTYPE[x.dtype]
        new = lambda *shape, dtype=x.dtype: torch.empty(shape, dtype=dtype, device=x.device)  # noqa: E731
        seed = int(torch.randint(0, 2 ** 62, (1,)))

        # weights: per-tile abs-max (ADC bound, noise scales) and the noisy copy
        w_noise = training and mod.noise_type.name != "NONE"
        noise_id = {"NONE": AHL_NOISE_NONE, "ADD_NORMAL": AHL_NOISE_ADD_NORMAL,
                    "ADD_NORMAL_PER_CHANNEL": AHL_NOISE_ADD_NORMAL_PER_CHANNEL}[mod.noise_type.name]
        mcfg = AhlModifierCfg(dt, 0, noise_id if w_noise else 0, 1.0, float(mod.std_dev), 0, 0, seed, 1, None)
        wmax, tile_max, tile_min = new(n_tiles, n_out), new(n_tiles, dtype=torch.float32), \
            new(n_tiles, dtype=torch.float32)
        w_eff = new(n_out, k_in) if w_noise else w
        _ok(lib.ahl_weight_prep(_p(w), n_out, k_in, k_in, ends, n_tiles, byref(mcfg), _p(wmax),
                                _p(tile_max), _p(tile_min), _p(w_eff) if w_noise else None, k_in,
                                stream), "ahl_weight_prep")

        ir_mode = AHL_IR_NONE if not irp.enable else (AHL_IR_DYNAMIC if irp.dynamic else AHL_IR_STATIC)
        per_channel = "PER_CHANNEL" in rpu_config.clip.type.name
        cfg = AhlLinearCfg(dt, ir_mode, fwd.inp_res, fwd.out_res, fwd.out_bound,
                           fwd.out_noise if training else 0.0, int(fwd.out_noise_per_channel),
                           int(per_channel), int(training), 0, irp.decay, irp.input_min_percentage,
                           0, 0, seed % 0xFFFFFFFF + 1, seed, 0, None)   # flag_token: new per call
        # input: clamp to the range + DAC in one pass (the dynamic ranges come out of it)
        xq = new(m_rows, k_in)
        ir = input_range.detach().contiguous() if ir_mode == AHL_IR_STATIC else None
        ir_dyn = new(n_tiles, m_rows) if ir_mode == AHL_IR_DYNAMIC else None
        _ok(lib.ahl_dac(_p(x), k_in, _p(xq), k_in, _p(ir), _p(ir_dyn), m_rows, k_in, ends, n_tiles,
                        byref(cfg), stream), "ahl_dac")
        if ir_mode == AHL_IR_DYNAMIC:
            ir = ir_dyn
        # the product; the clamp mask and its flag are what the backward needs from it
        y = new(m_rows, n_out)
        mask = flag = None
        if fwd.out_bound > 0:
            mask = new(n_tiles, (n_out + 31) // 32, (m_rows + 63) // 64 * 64, dtype=torch.int32)
            flag = new(1, dtype=torch.int32)
        _ok(lib.ahl_linear_fwd(_p(x), k_in, _p(xq), k_in, _p(w_eff), k_in, None, _p(y), n_out,
                               _p(mask), _p(flag), _p(ir), _p(wmax), _p(tile_max), m_rows, k_in,
                               n_out, ends, n_tiles, byref(cfg), None, stream), "ahl_linear_fwd")
        ctx.save_for_backward(x, xq, w_eff, mask, flag, ir)
        ctx.call = (cfg, ends, n_tiles, ir_mode)
        ctx.inp_shape = inp.shape
        return y.view(*inp.shape[:-1], n_out)

    @staticmethod
    def backward(ctx, grad_out):
        # pylint: disable=arguments-differ
        lib = HipSlotLinear.LIB
        x, xq, w_eff, mask, flag, ir = ctx.saved_tensors
        cfg, ends, n_tiles, ir_mode = ctx.call
        g = grad_out.reshape(-1, grad_out.size(-1)).contiguous()
        m_rows, n_out = g.shape
        k_in = x.size(1)
        stream = c_void_p(torch.cuda.current_stream().cuda_stream)
        new = lambda *shape, dtype=g.dtype: torch.empty(shape, dtype=dtype, device=g.device)  # noqa: E731
        static = ir_mode == AHL_IR_STATIC
        dx, dw = new(m_rows, k_in), new(n_out, k_in)
        ir_grad = new(n_tiles) if static else None
        ws = new(max(1, lib.ahl_linear_bwd_dx_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype, 0)),
                 dtype=torch.uint8)
        _ok(lib.ahl_linear_bwd_dx(_p(g), n_out, _p(mask), _p(flag), _p(w_eff), k_in,
                                  _p(x) if static else None, k_in if static else 0, _p(ir), _p(dx), k_in,
                                  _p(ir_grad), m_rows, k_in, n_out, ends, n_tiles, byref(cfg),
                                  _p(ws), stream), "ahl_linear_bwd_dx")
        ws = new(max(1, lib.ahl_linear_bwd_dw_ws_bytes(m_rows, k_in, n_out, n_tiles, cfg.dtype,
                                                       0 if mask is None else 1, 0)), dtype=torch.uint8)
        _ok(lib.ahl_linear_bwd_dw(_p(g), n_out, _p(mask), _p(flag), None, 0, _p(xq), k_in, _p(ir),
                                  _p(dw), k_in, None, m_rows, k_in, n_out, ends, n_tiles, byref(cfg),
                                  _p(ws), stream), "ahl_linear_bwd_dw")
        return dx.view(ctx.inp_shape), dw, ir_grad, None, None, None, None, None


@pytest.fixture(scope="module")
def slot():
    HipSlotLinear.LIB = _load()
    return HipSlotLinear


def _config(ir_mode, noise):
    from aihwkit_lightning.simulator.configs import (
        TorchInferenceRPUConfig, WeightClipType, WeightNoiseInjectionType,
    )

    cfg = TorchInferenceRPUConfig()
    cfg.mapping.max_input_size = 128
    cfg.forward.inp_res, cfg.forward.out_res, cfg.forward.out_bound = 254, 254, 6.0
    cfg.forward.out_noise = 0.05 if noise else 0.0
    cfg.clip.type = WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
    cfg.clip.sigma = 2.5
    if noise:
        cfg.modifier.noise_type = WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL
        cfg.modifier.std_dev = 0.03
    ir = cfg.pre_post.input_range
    ir.enable, ir.dynamic, ir.learn_input_range = ir_mode != "none", ir_mode == "dynamic", True
    ir.init_value, ir.init_from_data, ir.decay, ir.input_min_percentage = 2.0, 0, 0.01, 0.95
    if ir_mode == "none":
        cfg.forward.inp_res = cfg.forward.out_res = -1
        cfg.forward.out_bound = -1
    return cfg


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("ir_mode", ["static", "dynamic", "none"])
def test_slot_binding_equals_the_layer(slot, dtype, ir_mode):
    from aihwkit_lightning.nn import AnalogLinear

    gen = torch.Generator().manual_seed(11)
    m_rows, k_in, n_out = 192, 384, 136
    cfg = _config(ir_mode, noise=False)
    layer = AnalogLinear(k_in, n_out, bias=False, dtype=dtype, rpu_config=cfg)
    layer.set_weights_and_biases((0.05 * torch.randn(n_out, k_in, generator=gen)).to(dtype), None)
    layer = layer.cuda().train()
    x = (1.2 * torch.randn(4, m_rows // 4, k_in, generator=gen)).to(dtype).cuda()
    g = torch.randn(4, m_rows // 4, n_out, generator=gen).to(dtype).cuda()

    x_layer = x.clone().requires_grad_(True)
    out_layer = layer(x_layer)
    out_layer.backward(g)
    want = (out_layer.detach(), x_layer.grad, layer.weight.grad,
            layer.input_range.grad if ir_mode == "static" else None)

    x_slot = x.clone().requires_grad_(True)
    w_slot = layer.weight.detach().clone().requires_grad_(True)
    ir_slot = layer.input_range.detach().clone().requires_grad_(True) if ir_mode == "static" else None
    ends = torch.tensor(layer.in_sizes).cumsum(0)
    out = slot.apply(x_slot, w_slot, ir_slot, layer.input_range_update_idx, None, ends, cfg, True)
    out.backward(g)
    got = (out.detach(), x_slot.grad, w_slot.grad, ir_slot.grad if ir_mode == "static" else None)
    for name, a, b in zip(("out", "dx", "dw", "d input_range"), got, want):
        if b is None:
            continue
        assert a.shape == b.shape, name
        assert torch.equal(a, b), f"{name}: {(a.float() - b.float()).abs().max().item()}"


def test_slot_binding_draws_noise_of_the_configured_size(slot):
    """Training mode with both noises: the output differs from call to call, and its spread
    around the noise-free output is the configured one (out_noise / sqrt(T) * range * max|W| per
    tile, reference torch_utils/torch_linear.py:255-283) to a few percent."""
    from aihwkit_lightning.nn import AnalogLinear

    gen = torch.Generator().manual_seed(5)
    m_rows, k_in, n_out = 2048, 256, 128
    cfg = _config("static", noise=True)
    cfg.modifier.std_dev = 0.0           # output noise only, so the spread has a closed form
    cfg.forward.out_res = -1
    cfg.forward.out_bound = 1e6
    layer = AnalogLinear(k_in, n_out, bias=False, dtype=torch.float32, rpu_config=cfg)
    layer.set_weights_and_biases(0.05 * torch.randn(n_out, k_in, generator=gen), None)
    layer = layer.cuda()
    x = torch.randn(m_rows, k_in, generator=gen).cuda()
    ends = torch.tensor(layer.in_sizes).cumsum(0)
    args = (x, layer.weight.detach(), layer.input_range.detach(), layer.input_range_update_idx, None,
            ends, cfg)
    clean = slot.apply(*args, False)
    one, two = slot.apply(*args, True), slot.apply(*args, True)
    assert not torch.equal(one, two)
    n_tiles = len(layer.in_sizes)
    w = layer.weight.detach()
    var = torch.zeros(n_out, device="cuda")
    start = 0
    for t, size in enumerate(layer.in_sizes):
        wmax = w[:, start:start + size].abs().max()   # not per channel: the tile's largest weight
        var += (cfg.forward.out_noise / n_tiles ** 0.5 * layer.input_range[t].item() * wmax) ** 2
        start += size
    measured = (one - clean).var(dim=0)
    assert torch.allclose(measured, var, rtol=0.15), (measured / var).aminmax()
    assert abs((measured / var).mean().item() - 1.0) < 0.02

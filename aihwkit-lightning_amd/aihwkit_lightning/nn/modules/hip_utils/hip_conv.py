"""``HipConv``: the analog convolution read off the image itself, without the patch matrix.

The reference's ``_AnalogConvNd.forward`` (``nn/modules/conv.py:310-360``) unfolds the input into
``[B * L, C * kvol]`` patches and runs the linear operator on them. For the configurations
:func:`direct_conv_applies` accepts (16-bit dtype, stride 1, dilation 1, a learned static input
range or none, K-tiles that hold whole channels in multiples of 64, out_channels a multiple of 64)
this function keeps the input as one zero-padded, channels-last matrix of pixel rows instead and
lets the three matrix kernels address it directly (``csrc/ahl_conv_direct.hip``): same model, same
per-tile arithmetic, no ``[B * L, C * kvol]`` tensor in either direction. Everything else takes the
patch path (``PatchRows`` -> ``HipLinear`` -> ``SwapLastTwo`` in ``conv.py``).
"""
from ctypes import byref, c_int64
from typing import List, Optional

import torch
from torch import Tensor
from torch.autograd import Function

from . import library as L
from . import ops
from .hip_linear import NOISE_IDS, QUANT_IDS, check_supported, draw_seed, next_flag_token
from ....exceptions import HipBackendError
from ....simulator.configs import (
    TorchInferenceRPUConfig,
    WeightClipType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
)

# the switch for comparisons: False sends every convolution down the patch path
ENABLED = True


def _check(status: int, where: str) -> None:
    L.check(status, where)


def direct_conv_applies(layer, inp: Tensor, geom: List[int], init_active: bool) -> bool:
    """Whether this call can run without the patch matrix."""
    if not ENABLED or inp.dtype not in (torch.bfloat16, torch.float16) or not inp.is_cuda:
        return False
    if inp.numel() == 0:
        return False
    cfg = layer.rpu_config
    ir = cfg.pre_post.input_range
    if ir.enable and (ir.dynamic or ir.fast_mode or init_active):
        return False
    if cfg.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL:
        return False
    if any(v != 1 for v in geom[8:11]) or any(v != 1 for v in geom[14:17]):
        return False
    weight = layer.weight_matrix()
    if weight.device != inp.device or weight.dtype != inp.dtype or not weight.is_contiguous():
        return False
    return bool(L.load().ahl_conv_direct_supported(
        byref(ops.conv_geom(geom)), ops.dtype_id(inp.dtype), weight.size(0),
        L.tile_ends_array(layer.in_sizes), len(layer.in_sizes)))


def _rows(geom) -> List[int]:
    pixels, lead, rows = c_int64(), c_int64(), c_int64()
    _check(L.load().ahl_conv_direct_rows(byref(geom), byref(pixels), byref(lead), byref(rows)),
           "ahl_conv_direct_rows")
    return [pixels.value, lead.value, rows.value]


class HipConv(Function):
    """``y = conv(x, W) + b`` through the analog tile model, on the padded pixel grid."""

    # pylint: disable=abstract-method, arguments-differ, too-many-locals, too-many-arguments

    @staticmethod
    def forward(ctx, inp: Tensor, weights: Tensor, bias: Optional[Tensor], input_range: Optional[Tensor],
                in_sizes: List[int], rpu_config: TorchInferenceRPUConfig, training: bool,
                geom: List[int]) -> Tensor:
        check_supported(rpu_config)
        lib = L.load()
        fwd, modifier = rpu_config.forward, rpu_config.modifier
        ir_params = rpu_config.pre_post.input_range
        dev, dtype = inp.device, inp.dtype
        n_out, k_in = weights.shape
        n_tiles = len(in_sizes)
        ends = L.tile_ends_array(in_sizes)
        cgeom = ops.conv_geom(geom)
        pixels, lead, rows = _rows(cgeom)
        channels = geom[1]
        ctx.inp_shape = inp.shape
        inp = inp.contiguous()

        if fwd.out_res > 0:
            assert fwd.out_bound > 0, "Out quant. without a bound."
            assert ir_params.enable, "Out quant. without IR."
        ir_mode = L.AHL_IR_STATIC if ir_params.enable else L.AHL_IR_NONE
        if ir_mode == L.AHL_IR_NONE:
            assert fwd.inp_res <= 0, "Input range must be provided"
        else:
            assert input_range is not None, "Input range must be provided"
        noise_on = training and fwd.out_noise > 0
        bound_on = fwd.out_bound > 0 or fwd.out_res > 0
        if noise_on or bound_on:
            assert ir_params.enable, "Input range must be enabled"
        w_noise = training and modifier.noise_type != WeightNoiseInjectionType.NONE
        w_quant = modifier.quantization_type != WeightQuantizationType.NONE
        need_wmax = bound_on or noise_on or w_noise or w_quant
        per_channel_bound = rpu_config.clip.type == WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL
        ir_needs_grad = ir_mode == L.AHL_IR_STATIC and input_range.requires_grad and ctx.needs_input_grad[3]
        need_dx = ctx.needs_input_grad[0] or ir_needs_grad
        need_dw = ctx.needs_input_grad[1]

        # the Philox key: drawn on the host or, while the stream is being captured into a graph,
        # the device noise state advanced by one recorded launch (as in HipLinear.forward)
        seed, state_ptr = 0, 0
        if noise_on or w_noise:
            if torch.cuda.is_current_stream_capturing():
                state = ops.noise_state(dev, create=False)
                if state is None:
                    raise HipBackendError(
                        "a noisy layer is being captured into a graph before the device noise "
                        "state exists: call aihwkit_lightning.nn.graphs.prepare_noise_state(device) "
                        "(or use graphed_module) before the capture"
                    )
                ops.seed_advance(state, 2)
                state_ptr = state.data_ptr()
            else:
                seed = draw_seed()
        wmax = tile_max = None
        w_eff = weights.detach()
        if need_wmax:
            skip_tile_stats = ((not bound_on or per_channel_bound)
                               and (not noise_on or fwd.out_noise_per_channel))
            wmax, tile_max, _, eff = ops.weight_prep(
                w_eff, in_sizes, QUANT_IDS[modifier.quantization_type],
                NOISE_IDS[modifier.noise_type] if w_noise else L.AHL_NOISE_NONE,
                float(modifier.res) if w_quant else 1.0, float(modifier.std_dev), seed, 1,
                w_noise or w_quant, skip_tile_stats, state_ptr,
            )
            if w_noise or w_quant:
                w_eff = eff
        icfg = [ir_mode, int(fwd.out_noise_per_channel), int(per_channel_bound), int(training),
                1 if ops.os_environ_no_rounding() else 0, seed, 0, L.AHL_IR_GRAD_LEARNED, 0, state_ptr,
                # 0 under capture: a token baked into a recording would match on every replay
                0 if torch.cuda.is_current_stream_capturing() else next_flag_token()]
        fcfg = [float(fwd.inp_res), float(fwd.out_res), float(fwd.out_bound),
                float(fwd.out_noise) if noise_on else 0.0, float(ir_params.decay),
                float(ir_params.input_min_percentage)]
        cfg = ops.linear_cfg(dtype, icfg, fcfg)
        stream = ops.current_stream()
        dt = ops.dtype_id(dtype)

        ir_dev = None
        if ir_mode == L.AHL_IR_STATIC:
            ir_dev = input_range.detach().contiguous()
        # the image as zero-padded channels-last pixel rows, quantised per K-tile on the way (the
        # entry point writes every row of the buffers, the zeros included); with a static range
        # and a backward pass to come also what that pass needs to know about x: the range flags
        # of every element and the clipped-entry counts
        xq_rows = torch.empty((rows, channels), dtype=dtype, device=dev)
        keep_flags = ir_mode == L.AHL_IR_STATIC and need_dx
        flag_rows = counts = None
        if keep_flags:
            flag_rows = torch.empty((rows, channels), dtype=torch.uint8, device=dev)
            counts = torch.empty((lib.ahl_conv_count_words(byref(cgeom)),), dtype=torch.int32, device=dev)
        _check(lib.ahl_conv_image_rows(ops.ptr(inp), byref(cgeom), dt, ops.ptr(ir_dev), ends, n_tiles,
                                       byref(cfg), ops.ptr(xq_rows), ops.ptr(flag_rows), ops.ptr(counts), stream),
               "ahl_conv_image_rows")
        # the forward's operand and, for a step that wants dx, the input gradient's in the same launch
        w_taps = torch.empty_like(w_eff)
        w_dx = None
        if need_dx:
            w_dx = torch.empty((channels, k_in // channels * n_out), dtype=dtype, device=dev)
            _check(lib.ahl_conv_weight_layouts(ops.ptr(w_eff), k_in, dt, n_out, byref(cgeom), ends, n_tiles,
                                               ops.ptr(w_taps), k_in, ops.ptr(w_dx), w_dx.size(1), stream),
                   "ahl_conv_weight_layouts")
        else:
            _check(lib.ahl_conv_weight_layout(ops.ptr(w_eff), k_in, dt, n_out, byref(cgeom), ends, n_tiles, 0, 0,
                                              ops.ptr(w_taps), k_in, stream), "ahl_conv_weight_layout")
        want_keep = fwd.out_bound > 0 and (need_dx or need_dw)
        y_rows = torch.empty((pixels, n_out), dtype=dtype, device=dev)
        keep = flag = None
        if want_keep:
            keep = torch.empty((n_tiles, (n_out + 31) // 32, (pixels + 63) // 64 * 64), dtype=torch.int32, device=dev)
            if pixels % 64 != 0:
                keep[:, :, pixels:].zero_()
            flag = torch.empty((1,), dtype=torch.int32, device=dev)
        bias_c = None if bias is None else bias.detach().contiguous()
        _check(lib.ahl_conv_fwd(ops.ptr(xq_rows), ops.ptr(w_taps), ops.ptr(bias_c), ops.ptr(y_rows), ops.ptr(keep),
                                ops.ptr(flag), ops.ptr(ir_dev), ops.ptr(wmax), ops.ptr(tile_max), byref(cgeom),
                                n_out, ends, n_tiles, byref(cfg), stream), "ahl_conv_fwd")
        out_size = ops.conv_out_size(geom)
        y = torch.empty((geom[0], n_out, *out_size), dtype=dtype, device=dev)
        _check(lib.ahl_conv_output(ops.ptr(y_rows), byref(cgeom), dt, n_out, ops.ptr(y), stream), "ahl_conv_output")

        ctx.geom, ctx.in_sizes, ctx.icfg, ctx.fcfg = geom, in_sizes, icfg, fcfg
        ctx.need_dx, ctx.need_dw, ctx.ir_needs_grad = need_dx, need_dw, ir_needs_grad
        ctx.ir_mode, ctx.has_bias = ir_mode, bias is not None
        ctx.save_for_backward(
            xq_rows if need_dw else None, flag_rows, counts,
            w_dx, keep, flag, ir_dev,
        )
        return y

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        xq_rows, flag_rows, counts, w_dx, keep, flag, ir_dev = ctx.saved_tensors
        lib = L.load()
        geom, in_sizes = ctx.geom, ctx.in_sizes
        cgeom = ops.conv_geom(geom)
        pixels, _, rows = _rows(cgeom)
        n_tiles = len(in_sizes)
        ends = L.tile_ends_array(in_sizes)
        g = grad_out.contiguous()
        dev, dtype = g.device, g.dtype
        n_out, channels = g.size(1), geom[1]
        k_in = channels * geom[5] * geom[6] * geom[7]
        cfg = ops.linear_cfg(dtype, ctx.icfg, ctx.fcfg)
        stream = ops.current_stream()
        dt = ops.dtype_id(dtype)
        grad_inp = grad_w = grad_b = grad_ir = None
        want_bias = ctx.has_bias and ctx.needs_input_grad[2]
        if ctx.need_dx or ctx.need_dw:
            g_rows = torch.empty((rows, n_out), dtype=dtype, device=dev)
            _check(lib.ahl_conv_grad_rows(ops.ptr(g), byref(cgeom), dt, n_out, ops.ptr(g_rows), stream),
                   "ahl_conv_grad_rows")
        if ctx.need_dw:
            padded = c_int64()
            ws_bytes = lib.ahl_conv_bwd_dw_ws_bytes(byref(cgeom), n_out, ends, n_tiles, byref(padded))
            if ws_bytes < 0:
                raise HipBackendError("ahl_conv_bwd_dw_ws_bytes: bad geometry")
            ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device=dev)
            dw_tiled = torch.empty((n_out, padded.value), dtype=dtype, device=dev)
            dbias = torch.empty((n_out,), dtype=dtype, device=dev) if want_bias else None
            _check(lib.ahl_conv_bwd_dw(ops.ptr(g_rows), ops.ptr(keep), ops.ptr(flag), ops.ptr(xq_rows),
                                       ops.ptr(dw_tiled), ops.ptr(dbias), byref(cgeom), n_out, ends, n_tiles,
                                       byref(cfg), ops.ptr(ws), stream), "ahl_conv_bwd_dw")
            grad_w = torch.empty((n_out, k_in), dtype=dtype, device=dev)
            _check(lib.ahl_conv_weight_layout(ops.ptr(dw_tiled), padded.value, dt, n_out, byref(cgeom), ends,
                                              n_tiles, 1, padded.value // n_tiles, ops.ptr(grad_w), k_in, stream),
                   "ahl_conv_weight_layout")
            if want_bias:
                grad_b = dbias
        elif want_bias:
            grad_b = g.flatten(2).sum(dim=(0, 2)).to(dtype)
        if ctx.need_dx:
            static = ctx.ir_mode == L.AHL_IR_STATIC
            ws_bytes = lib.ahl_conv_bwd_dx_ws_bytes(byref(cgeom), n_tiles)
            ws = torch.empty((max(ws_bytes, 16),), dtype=torch.uint8, device=dev)
            dimg = torch.empty((pixels, channels), dtype=dtype, device=dev)
            dx = torch.empty((geom[0], channels, geom[2], geom[3], geom[4]), dtype=dtype, device=dev)
            ir_grad = torch.empty((n_tiles,), dtype=dtype, device=dev) if static else None
            _check(lib.ahl_conv_bwd_dx(ops.ptr(g_rows), ops.ptr(keep), ops.ptr(flag), ops.ptr(w_dx),
                                       ops.ptr(flag_rows), ops.ptr(counts), ops.ptr(ir_dev), ops.ptr(dimg), ops.ptr(dx),
                                       ops.ptr(ir_grad), byref(cgeom), n_out, ends, n_tiles, byref(cfg),
                                       ops.ptr(ws), stream), "ahl_conv_bwd_dx")
            if ctx.needs_input_grad[0]:
                grad_inp = dx.view(ctx.inp_shape)
            if ctx.ir_needs_grad:
                grad_ir = ir_grad
        return grad_inp, grad_w, grad_b, grad_ir, None, None, None, None

"""``HipLinear``: the autograd function that occupies the accelerated-operator slot of
``AnalogLinear.forward`` (the place of ``TritonLinear`` in the reference,
``nn/modules/linear.py:120-135`` / ``triton_utils/triton_linear.py:446-764``), with the
semantics of the reference's torch-mode (``torch_utils/torch_linear.py:116-314``).
"""
import itertools
import os
from typing import List, Optional

import torch
from torch import Tensor
from torch.autograd import Function

from . import library as L
from . import ops as _impl
from .ops import tile_stride
from ....exceptions import ConfigError, HipBackendError
from ....simulator.configs import (
    TorchInferenceRPUConfig,
    WeightClipType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
)

NOISE_IDS = {
    WeightNoiseInjectionType.NONE: L.AHL_NOISE_NONE,
    WeightNoiseInjectionType.ADD_NORMAL: L.AHL_NOISE_ADD_NORMAL,
    WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL: L.AHL_NOISE_ADD_NORMAL_PER_CHANNEL,
}
QUANT_IDS = {
    WeightQuantizationType.NONE: L.AHL_QUANT_NONE,
    WeightQuantizationType.DISCRETIZE: L.AHL_QUANT_DISCRETIZE,
    WeightQuantizationType.DISCRETIZE_PER_CHANNEL: L.AHL_QUANT_DISCRETIZE_PER_CHANNEL,
}


def draw_seed() -> int:
    """One Philox key per call from torch's CPU generator, so ``torch.manual_seed`` makes runs
    reproducible (the reference seeds its kernels the same way, ``triton_linear.py:541,617``)."""
    return int(torch.randint(0, 2**62, (1,)).item())


def check_supported(rpu_config: TorchInferenceRPUConfig) -> None:
    """Reject configuration combinations the reference rejects too."""
    if rpu_config.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL:
        # torch_utils/torch_linear.py:234-238
        assert rpu_config.modifier.quantization_type in (
            WeightQuantizationType.NONE, WeightQuantizationType.DISCRETIZE_PER_CHANNEL,
        ), "You can't learn weight ranges per column but quantize per tensor"


# bf16 products of at least this many multiply-adds get their output channels padded to a
# multiple of 8 (see HipLinear.forward); below it the general kernels are as fast
PAD_CHANNELS_MIN_WORK = 1 << 22


# Where HipLinear takes its operator calls from: it is an autograd node of its own, so inside it
# the dispatcher adds nothing but time (three to six calls per layer call)
_ops_for = _impl.direct


# dtypes with MFMA kernels of their own (two-byte elements); float32 runs on the general kernels
MFMA16_DTYPES = (torch.bfloat16, torch.float16)

_FLAG_TOKENS = itertools.count(1)


def next_flag_token() -> int:
    """A non-zero 32-bit value that differs from call to call (``AhlLinearCfg.flag_token``)."""
    return next(_FLAG_TOKENS) % 0xFFFFFFFF + 1


class HipLinear(Function):
    """y = analog_mvm(x, W) + b with DAC/ADC, noise and tiling, on MI355X."""

    # pylint: disable=abstract-method, arguments-differ, too-many-locals, too-many-arguments

    @staticmethod
    def forward(
        ctx,
        inp: Tensor,
        weights: Tensor,
        bias: Optional[Tensor],
        input_range: Optional[Tensor],
        input_range_update_idx: Optional[Tensor],
        in_sizes: List[int],
        rpu_config: TorchInferenceRPUConfig,
        training: bool,
        init_active: bool,
        x_min: Optional[Tensor] = None,
        x_max: Optional[Tensor] = None,
        learnable_weight_clip: Optional[Tensor] = None,
        weight_cache: Optional[dict] = None,
    ) -> Tensor:
        if not inp.is_cuda:
            raise HipBackendError(
                "AnalogLinear runs only on a ROCm device (got a CPU tensor); there is no CPU path"
            )
        check_supported(rpu_config)
        ops = _ops_for(inp)
        fwd, modifier = rpu_config.forward, rpu_config.modifier
        ir_params = rpu_config.pre_post.input_range
        k_in, n_out = weights.size(1), weights.size(0)
        out_shape = inp.shape[:-1] + (n_out,)
        x2 = inp.reshape(-1, k_in)
        if x2.stride(-1) != 1:
            x2 = x2.contiguous()
        weights_c = weights if weights.stride(1) == 1 else weights.contiguous()
        if weights.dtype != inp.dtype:
            raise HipBackendError("input and weight dtypes differ")
        if weights.device != inp.device or (bias is not None and bias.device != inp.device):
            raise HipBackendError(
                f"input on {inp.device} but parameters on {weights.device}: move the layer to the "
                "input's device"
            )
        m_rows = x2.size(0)

        apply_out_quantization = fwd.out_res > 0
        if apply_out_quantization:
            assert fwd.out_bound > 0, "Out quant. without a bound."
            assert ir_params.enable, "Out quant. without IR."
        # fast_mode takes precedence over dynamic, as in the reference (torch_linear.py:138-153)
        fast = bool(ir_params.enable and ir_params.fast_mode)
        if fast:
            assert x_min is not None, "x_min must be provided"
            assert x_max is not None, "x_max must be provided"
            assert input_range is not None, "Input range must be provided"
            assert input_range_update_idx is not None, "Input range update index must be provided"
            ir_mode = L.AHL_IR_STATIC
        elif ir_params.enable and not ir_params.dynamic:
            assert input_range is not None, "Input range must be provided"
            assert input_range_update_idx is not None, "Input range update index must be provided"
            ir_mode = L.AHL_IR_STATIC
        elif ir_params.enable:
            ir_mode = L.AHL_IR_DYNAMIC
        else:
            ir_mode = L.AHL_IR_NONE
            assert fwd.inp_res <= 0, "Input range must be provided"
        noise_on = training and fwd.out_noise > 0
        if noise_on:
            assert ir_params.enable, "Input range must be enabled"
        bound_on = fwd.out_bound > 0 or apply_out_quantization
        if bound_on:
            assert ir_params.enable, (
                "Input range must be provided when using an out_bound or out quantization"
            )
        w_noise = training and modifier.noise_type != WeightNoiseInjectionType.NONE
        w_quant = modifier.quantization_type != WeightQuantizationType.NONE
        learned_clip = rpu_config.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL
        if learned_clip:
            assert learnable_weight_clip is not None, "learnable_weight_clip should not be None"
        need_wmax = bound_on or noise_on or w_noise or w_quant or learned_clip
        per_channel_bound = rpu_config.clip.type in (WeightClipType.LAYER_GAUSSIAN_PER_CHANNEL,
                                                     WeightClipType.LEARNABLE_PER_CHANNEL)
        # the clip's gradient comes out of the weight gradient
        clip_needs_grad = learned_clip and ctx.needs_input_grad[11]
        ir_needs_grad = ir_mode == L.AHL_IR_STATIC and input_range.requires_grad
        need_dx = ctx.needs_input_grad[0] or (ctx.needs_input_grad[3] and ir_needs_grad)
        need_dw = ctx.needs_input_grad[1] or clip_needs_grad

        # One Philox seed per call from the host generator -- or, while the stream is being
        # captured into a HIP graph, the device-resident noise state advanced by one recorded
        # launch per call, so that every replay draws new noise.
        seed, state_ptr = 0, 0
        if (noise_on or w_noise) and m_rows > 0:
            if torch.cuda.is_current_stream_capturing():
                state = _impl.noise_state(inp.device, create=False)
                if state is None:
                    raise HipBackendError(
                        "a noisy layer is being captured into a graph before the device noise "
                        "state exists: call aihwkit_lightning.nn.graphs.prepare_noise_state(device) "
                        "(or use graphed_module) before the capture"
                    )
                _impl.seed_advance(state, 2)
                state_ptr = state.data_ptr()
            else:
                seed = draw_seed()
        wmax = tile_max = tile_min = None
        w_eff = weights_c
        clip_quant = L.AHL_QUANT_DISCRETIZE_PER_CHANNEL if w_quant else L.AHL_QUANT_CLIP_LEARNED
        if m_rows > 0 and learned_clip:
            # the clipped (+ quantised, + noisy) weights; the clip is the tile's "wmax" from here on
            wmax = learnable_weight_clip.detach()
            if not wmax.is_contiguous():
                wmax = wmax.contiguous()
            tile_max, tile_min, w_eff = ops.weight_prep_clip(
                weights_c, wmax, in_sizes, clip_quant,
                NOISE_IDS[modifier.noise_type] if w_noise else L.AHL_NOISE_NONE,
                float(modifier.res) if w_quant else 1.0, float(modifier.std_dev), seed, 1, state_ptr,
            )
        elif m_rows > 0 and need_wmax:
            res = float(modifier.res) if w_quant else 1.0
            # per-tile maxima are only read when the ADC bound or the output noise scale with
            # the whole tile instead of the channel
            skip_tile_stats = ((not bound_on or per_channel_bound)
                               and (not noise_on or fwd.out_noise_per_channel))
            # A caller that promises unchanged weights over several calls (the steps of a
            # recurrent sequence) passes a dict: what depends on the weights alone is computed
            # by the first call and reused. A modifier draws new weights per call: no reuse.
            reuse = weight_cache if not (w_noise or w_quant) else None
            stats_key = ("stats", skip_tile_stats)
            if reuse is not None and stats_key in reuse:
                wmax, tile_max = reuse[stats_key]
            else:
                wmax, tile_max, _, eff = ops.weight_prep(
                    weights_c, in_sizes, QUANT_IDS[modifier.quantization_type],
                    NOISE_IDS[modifier.noise_type] if w_noise else L.AHL_NOISE_NONE, res,
                    float(modifier.std_dev), seed, 1, w_noise or w_quant, skip_tile_stats, state_ptr,
                )
                if w_noise or w_quant:
                    w_eff = eff
                if reuse is not None:
                    reuse[stats_key] = (wmax, tile_max)

        # 16-bit layers whose output width is not a multiple of 8 (a 50257-word vocabulary): the
        # MFMA kernels handle channels in whole 16-byte vectors, so the weight-side operands get
        # zero channels up to the next multiple of 8 and the extra output columns are dropped.
        # (Their per-channel abs-max is set to 1 so that their ADC step is not 0; nothing of them
        # reaches the result.) Small problems stay on the general kernels: the copies would cost
        # more than they save.
        pad_n = 0
        bias_k = bias
        if (inp.dtype in MFMA16_DTYPES and n_out % 8 != 0 and not learned_clip
                and m_rows * k_in * n_out >= PAD_CHANNELS_MIN_WORK):
            pad_n = 8 - n_out % 8
            frozen = weight_cache if w_eff is weights_c else None  # no per-call modifier
            if frozen is not None and ("channels", pad_n) in frozen:
                w_eff, wmax, bias_k = frozen[("channels", pad_n)]
            else:
                w_eff = torch.nn.functional.pad(w_eff.detach(), (0, 0, 0, pad_n))
                if wmax is not None:
                    wmax = torch.nn.functional.pad(wmax, (0, pad_n), value=1.0)
                if bias is not None:
                    bias_k = torch.nn.functional.pad(bias.detach(), (0, pad_n))
                if frozen is not None:
                    frozen[("channels", pad_n)] = (w_eff, wmax, bias_k)
        n_k = n_out + pad_n
        weights_frozen = weight_cache is not None and not (w_noise or w_quant or learned_clip)

        # 16-bit splits whose tiles do not start on the MFMA kernels' 256-column block boundaries:
        # the quantised input and the effective weights are kept in a padded tile layout instead
        # (stride > 0), unless the padding would blow the work up more than the slower general
        # kernels do, or the shape does not fit the fast backward at all
        stride = 0
        dense_fwd_ok = len(set(in_sizes)) == 1 and in_sizes[0] % 64 == 0
        if (inp.dtype in MFMA16_DTYPES and m_rows > 0 and n_k % 8 == 0
                and w_eff.data_ptr() % 16 == 0):
            stride = tile_stride(k_in, len(in_sizes), inp.dtype)
            if stride * len(in_sizes) > 4 * k_in or (dense_fwd_ok and not (need_dx or need_dw)):
                stride = 0

        skip_rounding = 1 if os.environ.get("_AIHWKIT_NO_ROUNDING", False) else 0
        icfg = [
            ir_mode, int(fwd.out_noise_per_channel), int(per_channel_bound),
            int(training), skip_rounding, seed, 0,
            # fast_mode clamps with torch.clamp: its autograd rule instead of the learned-range one
            L.AHL_IR_GRAD_CLAMP if fast else L.AHL_IR_GRAD_LEARNED,
            stride,
            state_ptr,
            # what "something was clamped" looks like in this call's one-word flag: a value of
            # its own per call, so that the forward need not clear the word first. A call that is
            # being recorded into a graph passes 0 instead (the library's own clearing launch is
            # recorded): a token baked into the recording would be the same on every replay, and
            # after the first replay that clamps every later one would find a stale match
            0 if torch.cuda.is_current_stream_capturing() else next_flag_token(),
        ]
        fcfg = [
            float(fwd.inp_res), float(fwd.out_res), float(fwd.out_bound),
            float(fwd.out_noise) if noise_on else 0.0, float(ir_params.decay),
            float(ir_params.input_min_percentage),
        ]
        ctx.empty = m_rows == 0
        if ctx.empty:
            # no rows: zero gradients for everything that asks for one (the reference returns
            # zeros here too, e.g. for a routed expert that received no token in a step)
            ctx.zero_like = [t if (t is not None and need) else None for t, need in zip(
                (inp, weights, bias, input_range, learnable_weight_clip),
                (ctx.needs_input_grad[i] for i in (0, 1, 2, 3, 11)))]
            return inp.new_zeros(out_shape)

        # 16-bit dtypes with equal tiles of a multiple of 64 inputs: clamp + DAC (+ dynamic abs-max) run as
        # one memory-bound pass and the matrix kernel streams the quantised input; otherwise the
        # clamp + DAC are fused into the matrix kernel's A-tile staging.
        split_dac = stride > 0 or (inp.dtype in MFMA16_DTYPES and dense_fwd_ok and n_k % 8 == 0)
        if stride > 0:
            tiles_key = ("tiles", stride, pad_n)
            if weights_frozen and tiles_key in weight_cache:
                w_eff = weight_cache[tiles_key]
            else:
                w_eff = ops.pad_tiles(w_eff, in_sizes, stride)
                if weights_frozen:
                    weight_cache[tiles_key] = w_eff
        ir_dev = xq = None
        if ir_mode == L.AHL_IR_STATIC:
            if training and init_active and fast:
                ops.ir_fast_update(
                    x2, in_sizes, input_range.data, input_range_update_idx, x_min, x_max,
                    float(ir_params.init_from_data), float(ir_params.act_range_momentum),
                )
            elif training and init_active:
                std = ops.sliced_std(x2, in_sizes)
                ops.ir_init_update(
                    input_range.data, input_range_update_idx, std, float(ir_params.init_from_data),
                    float(ir_params.init_std_alpha),
                )
            ir_dev = input_range.detach()
            if not ir_dev.is_contiguous():
                ir_dev = ir_dev.contiguous()
        if split_dac:
            xq, ir_dyn = ops.dac(x2, ir_dev, in_sizes, icfg, fcfg)
            if ir_mode == L.AHL_IR_DYNAMIC:
                ir_dev = ir_dyn
        elif ir_mode == L.AHL_IR_DYNAMIC:
            ir_dev = ops.sliced_absmax(x2, in_sizes, False)[0]

        want_keep = fwd.out_bound > 0 and (need_dx or need_dw)
        y, keep, flag = ops.linear_fwd(
            # x goes along with xq: should the MFMA kernel not apply after all (a misaligned
            # view), the general kernel starts from x
            x2 if (stride == 0 or not split_dac) else None, xq, w_eff, bias_k, ir_dev, wmax, tile_max,
            in_sizes, icfg, fcfg,
            want_keep,
        )
        if pad_n:
            y = y[:, :n_out]
        ctx.pad_n = pad_n

        ctx.in_sizes, ctx.icfg, ctx.fcfg = in_sizes, icfg, fcfg
        ctx.inp_shape, ctx.ir_mode, ctx.has_bias = inp.shape, ir_mode, bias is not None
        ctx.need_dx, ctx.need_dw, ctx.ir_needs_grad = need_dx, need_dw, ir_needs_grad
        ctx.learned_clip = learned_clip and need_dw
        ctx.clip_quant, ctx.clip_res = clip_quant, float(modifier.res) if w_quant else 1.0
        need_x = (need_dx and ir_mode == L.AHL_IR_STATIC) or (need_dw and xq is None)
        ctx.save_for_backward(
            x2 if need_x else None, xq if need_dw else None,
            (w_eff if w_eff is not weights else weights.detach()) if need_dx else None,
            keep if want_keep else None, flag if want_keep else None,
            # while the range is still initialised from data, the next forward rewrites it in
            # place (possibly before this call's backward): keep this call's values then
            ir_dev.clone() if (ir_mode == L.AHL_IR_STATIC and init_active) else ir_dev,
            weights_c.detach() if ctx.learned_clip else None,
            wmax.clone() if ctx.learned_clip else None, tile_min if ctx.learned_clip else None,
        )
        return y.view(out_shape)

    @staticmethod
    def backward(ctx, grad_out: Tensor):
        if ctx.empty:
            d_inp, d_w, d_b, d_ir, d_clip = (None if t is None else torch.zeros_like(t)
                                             for t in ctx.zero_like)
            return (d_inp, d_w, d_b, d_ir, None, None, None, None, None, None, None, d_clip, None)
        x2, xq, w_eff, keep, flag, ir_dev, w_plain, clip, clip_tile_min = ctx.saved_tensors
        n_out = grad_out.size(-1)
        g2 = grad_out.reshape(-1, n_out)
        if g2.stride(-1) != 1 or (g2.size(0) > 1 and g2.stride(0) != n_out):
            g2 = g2.contiguous()
        grad_inp = grad_w = grad_b = grad_ir = grad_clip = None
        ops = _ops_for(g2)
        g_plain = g2
        if ctx.pad_n and (ctx.need_dx or ctx.need_dw):
            g2 = torch.nn.functional.pad(g2, (0, ctx.pad_n))  # zero gradient for the extra channels
        if ctx.need_dx:
            dx, ir_grad = ops.linear_bwd_dx(
                g2, keep, flag, w_eff, x2 if ctx.ir_mode == L.AHL_IR_STATIC else None, ir_dev,
                ctx.in_sizes, ctx.icfg, ctx.fcfg,
            )
            if ctx.needs_input_grad[0]:
                grad_inp = dx.view(ctx.inp_shape)
            if ctx.ir_needs_grad and ctx.needs_input_grad[3]:
                grad_ir = ir_grad
        want_bias = ctx.has_bias and ctx.needs_input_grad[2]
        if ctx.need_dw:
            # the weight-gradient kernel streams all of g and sums its columns on the way
            grad_w, dbias = ops.linear_bwd_dw(
                g2, keep, flag, x2 if xq is None else None, xq, ir_dev, ctx.in_sizes, ctx.icfg,
                ctx.fcfg, want_bias,
            )
            if ctx.pad_n:
                grad_w = grad_w[:n_out]
                dbias = dbias[:n_out] if want_bias else dbias
            if want_bias:
                grad_b = dbias
            if ctx.learned_clip:
                # gradient w.r.t. the clipped weights -> weights (in place) and clip (LSQ rule)
                grad_clip = ops.learned_clip_bwd(
                    grad_w, w_plain, clip, clip_tile_min, ctx.in_sizes, ctx.clip_quant, ctx.clip_res
                )
        elif want_bias:
            grad_b = ops.col_sum(g_plain)
        if not ctx.needs_input_grad[1]:
            grad_w = None
        return (grad_inp, grad_w, grad_b, grad_ir, None, None, None, None, None, None, None,
                grad_clip, None)

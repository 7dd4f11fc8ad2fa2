"""Post-training calibration of the input ranges (reference
``inference/calibration/calibration.py:36-319``). The ``MAX`` strategy runs on the device as a
running per-tile abs-max, the moving strategies as a per-batch std or exact quantile (radix
selection) plus a device-side moving average, the cached-quantile strategy as a row cache on
the device; no strategy synchronises with the host per batch."""
from copy import deepcopy
from enum import Enum
from functools import partial
from typing import Dict, Iterator, List, Optional, Tuple

import torch
from torch import Tensor, no_grad
from torch.nn import Parameter
from torch.utils.hooks import RemovableHandle

from ...exceptions import ConfigError
from ...nn import AnalogLinear
from ...nn.modules.conv import _AnalogConvNd
from ...nn.modules.hip_utils.ops import OPS, direct
from ...simulator.configs import TorchInferenceRPUConfig, WeightNoiseInjectionType


class InputRangeCalibrationType(Enum):
    """How the per-tile input range is derived from calibration data."""

    NONE = "None"
    MOVING_STD = "MovingStd"
    MOVING_QUANTILE = "MovingQuantile"
    CACHE_QUANTILE = "CacheQuantile"
    MAX = "Max"


def _tile_rows(mod, args: Tuple, kwargs: Dict) -> Tensor:
    """The rows ``[n, in_features]`` the tiles of ``mod`` see for this call."""
    x_input: Tensor = args[0] if len(args) > 0 else kwargs["inp"]
    if isinstance(mod, _AnalogConvNd):
        # the tiles of a convolution see patches, not the image (reference calibration.py:82-93)
        x_input = mod.patch_rows(x_input)
    return x_input.reshape(-1, x_input.size(-1))


def _calibration_pre_forward(mod, args: Tuple, kwargs: Dict, calibration_type, cache: Dict,
                             key: str, max_samples: int, ir_quantile: float) -> None:
    """Forward pre-hook: fold this batch into the layer's calibration state (reference
    ``calibration.py:57-152``). Everything stays on the device. ``MAX`` and the two moving
    strategies never wait for it; ``CACHE_QUANTILE`` does once per batch (the number of rows
    that are not all zero decides a tensor shape) and keeps up to ``max_samples`` fp32 rows of
    ``in_features`` values per layer in device memory, where the reference keeps them on the host."""
    x_input = _tile_rows(mod, args, kwargs)
    if x_input.size(0) == 0:
        return
    OPS = direct(x_input)   # a hook is never traced: the operators without the dispatcher hop  # noqa: N806
    ir_params = mod.rpu_config.pre_post.input_range
    if calibration_type == InputRangeCalibrationType.MAX:
        if key not in cache:
            cache[key] = torch.full((len(mod.in_sizes),), float("-inf"), dtype=torch.float32,
                                    device=x_input.device)
        OPS.running_absmax(x_input, mod.in_sizes, cache[key])
    elif calibration_type == InputRangeCalibrationType.CACHE_QUANTILE:
        # keep at most max_samples of the rows that are not all zero, re-drawn with torch's CPU
        # generator after every batch like the reference (calibration.py:104-110); the rows stay
        # on the device
        rows = x_input[OPS.row_nonzero(x_input).bool()].float()
        merged = rows if key not in cache else torch.cat([cache[key], rows])
        pick = torch.randperm(merged.size(0))[:max_samples]
        cache[key] = merged[pick.to(merged.device)]
    elif calibration_type == InputRangeCalibrationType.MOVING_STD:
        stat = OPS.sliced_std_kept(x_input, mod.in_sizes)
        OPS.ir_moving_update(mod.input_range.data, mod.input_range_update_idx.data, stat,
                             float(ir_params.init_std_alpha), True)
    elif calibration_type == InputRangeCalibrationType.MOVING_QUANTILE:
        if ir_quantile == 1.0:
            stat = torch.full((len(mod.in_sizes),), float("-inf"), dtype=torch.float32,
                              device=x_input.device)
            OPS.running_absmax(x_input, mod.in_sizes, stat)
        else:
            stat = OPS.sliced_quantile(x_input, mod.in_sizes, float(ir_quantile))
        OPS.ir_moving_update(mod.input_range.data, mod.input_range_update_idx.data, stat, 1.0, False)
    else:
        raise ConfigError(f"Unknown InputRangeCalibrationType {calibration_type}")


@no_grad()
def calibrate_input_ranges(
    model,
    calibration_type: InputRangeCalibrationType,
    dataloader: Iterator,
    quantile: float = 0.99995,
    max_samples: int = 1000,
    std_alpha: Optional[float] = None,
    verbose: bool = True,
) -> None:
    """Stream ``(args, kwargs)`` pairs from ``dataloader`` through ``model`` (eval mode, input
    range disabled, no DAC) and set every analog layer's ``input_range`` from the statistics of
    the chosen strategy (reference ``calibration.py:155-319``); afterwards the input range is
    enabled and its data initialisation is marked finished.

    ``MAX``: abs-max of all inputs. ``CACHE_QUANTILE``: ``quantile`` of up to ``max_samples``
    cached rows. ``MOVING_STD`` / ``MOVING_QUANTILE``: the range starts at 3.0, is enabled while
    the data streams through, and follows the running mean of ``std_alpha`` standard deviations /
    of the per-batch ``quantile``.
    """
    # pylint: disable=too-many-locals, too-many-branches
    if calibration_type in (None, InputRangeCalibrationType.NONE) or not isinstance(
        calibration_type, InputRangeCalibrationType
    ):
        raise ConfigError(f"Unknown InputRangeCalibrationType {calibration_type}")
    sample_layer = next(model.analog_layers())
    rpu_config: TorchInferenceRPUConfig = sample_layer.rpu_config
    if rpu_config.pre_post.input_range.enable:
        raise ConfigError(
            "You can only calibrate input ranges for models that don't have input ranges."
        )
    if rpu_config.forward.inp_res > 0:
        raise ConfigError(
            "When calibrating the input ranges, the input res must be infinite (-1 or 0)"
        )
    if sample_layer.training:
        raise ConfigError("Calibration can only be done in test mode.")
    moving = calibration_type in (InputRangeCalibrationType.MOVING_QUANTILE,
                                  InputRangeCalibrationType.MOVING_STD)

    cache: Dict[str, Tensor] = {}
    saved_configs: Dict[str, TorchInferenceRPUConfig] = {}
    handles: List[RemovableHandle] = []
    for name, layer in model.named_analog_layers():
        weight = layer.weight
        if moving:
            # the range is live while the data streams through (calibration.py:228-250)
            ir_params = layer.rpu_config.pre_post.input_range
            ir_params.enable, ir_params.dynamic, ir_params.learn_input_range = True, False, True
            ir_params.init_value = 3.0
            if std_alpha is not None:
                ir_params.init_std_alpha = std_alpha
            layer.input_range = Parameter(
                torch.full((len(layer.in_sizes),), 3.0, dtype=weight.dtype, device=weight.device),
                requires_grad=True,
            )
            layer.input_range_update_idx = Parameter(
                torch.zeros((len(layer.in_sizes),), dtype=torch.int32, device=weight.device),
                requires_grad=False,
            )
            layer._ir_init_active = False  # pylint: disable=protected-access
        saved_configs[name] = deepcopy(layer.rpu_config)
        layer.rpu_config.forward.out_noise = 0.0
        layer.rpu_config.modifier.noise_type = WeightNoiseInjectionType.NONE
        hook = partial(_calibration_pre_forward, calibration_type=calibration_type, cache=cache,
                       key=name, max_samples=max_samples, ir_quantile=quantile)
        handles.append(layer.register_forward_pre_hook(hook, with_kwargs=True))

    if verbose:
        from tqdm import tqdm  # pylint: disable=import-outside-toplevel

        dataloader = tqdm(dataloader)
    for args, kwargs in dataloader:
        model(*args, **kwargs)
    for handle in handles:
        handle.remove()

    for name, layer in model.named_analog_layers():
        weight = layer.weight
        config = saved_configs[name]
        layer.input_range_update_idx = Parameter(
            torch.full((len(layer.in_sizes),), float("-inf"), device=weight.device, dtype=weight.dtype),
            requires_grad=False,
        )
        if not moving:
            config.pre_post.input_range.enable = True
            stats = cache.get(name)
            if stats is None:
                raise ConfigError(f"layer {name} saw no calibration data")
            if calibration_type == InputRangeCalibrationType.CACHE_QUANTILE:
                stats = OPS.sliced_quantile(stats, layer.in_sizes, float(quantile))
            layer.input_range = Parameter(
                stats.to(dtype=weight.dtype),
                requires_grad=config.pre_post.input_range.learn_input_range,
            )
        layer.rpu_config = config
        layer._ir_init_active = False  # pylint: disable=protected-access

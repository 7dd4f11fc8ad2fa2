"""Post-training calibration of the input ranges (reference
``inference/calibration/calibration.py:36-319``). The ``MAX`` strategy runs on the device as a
running per-tile abs-max with no host synchronisation per batch; the quantile and moving-std
strategies of the reference are not part of this build and raise ``ConfigError``."""
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
from ...nn.modules.hip_utils.ops import OPS
from ...simulator.configs import TorchInferenceRPUConfig, WeightNoiseInjectionType


class InputRangeCalibrationType(Enum):
    """How the per-tile input range is derived from calibration data."""

    NONE = "None"
    MOVING_STD = "MovingStd"
    MOVING_QUANTILE = "MovingQuantile"
    CACHE_QUANTILE = "CacheQuantile"
    MAX = "Max"


def _max_pre_forward(mod: AnalogLinear, args: Tuple, kwargs: Dict, cache: Dict[str, Tensor],
                     key: str) -> None:
    """Forward pre-hook: fold this batch into the layer's running per-tile abs-max."""
    x_input: Tensor = args[0] if len(args) > 0 else kwargs["inp"]
    if isinstance(mod, _AnalogConvNd):
        # the tiles of a convolution see patches, not the image (reference calibration.py:82-93)
        x_input = mod.patch_rows(x_input)
    x_input = x_input.reshape(-1, x_input.size(-1))
    if key not in cache:
        cache[key] = torch.full((len(mod.in_sizes),), float("-inf"), dtype=torch.float32,
                                device=x_input.device)
    if x_input.size(0) > 0:
        OPS.running_absmax(x_input, mod.in_sizes, cache[key])


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
    range disabled, no DAC) and set every analog layer's ``input_range`` from the statistics;
    afterwards the input range is enabled and its data initialisation is marked finished."""
    # pylint: disable=unused-argument, too-many-locals
    if calibration_type != InputRangeCalibrationType.MAX:
        raise ConfigError(
            f"{calibration_type} is not implemented by the HIP backend (only MAX is)"
        )
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

    cache: Dict[str, Tensor] = {}
    saved_configs: Dict[str, TorchInferenceRPUConfig] = {}
    handles: List[RemovableHandle] = []
    for name, layer in model.named_analog_layers():
        saved_configs[name] = deepcopy(layer.rpu_config)
        layer.rpu_config.forward.out_noise = 0.0
        layer.rpu_config.modifier.noise_type = WeightNoiseInjectionType.NONE
        hook = partial(_max_pre_forward, cache=cache, key=name)
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
        config.pre_post.input_range.enable = True
        layer.input_range_update_idx = Parameter(
            torch.full((len(layer.in_sizes),), float("-inf"), device=weight.device),
            requires_grad=False,
        )
        stats = cache.get(name)
        if stats is None:
            raise ConfigError(f"layer {name} saw no calibration data")
        layer.input_range = Parameter(
            stats.to(dtype=weight.dtype), requires_grad=config.pre_post.input_range.learn_input_range
        )
        layer.rpu_config = config
        layer._ir_init_active = False  # pylint: disable=protected-access

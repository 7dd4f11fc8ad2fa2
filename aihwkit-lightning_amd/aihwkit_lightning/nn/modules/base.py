"""Mixin shared by all analog layers: iteration over analog layers, input-range state,
deprecated-config migration. Parameter and buffer names, shapes and dtypes follow the reference
(``nn/modules/base.py:29-212``) so that checkpoints are interchangeable."""
import warnings
from typing import Any, Callable, Generator, List, Tuple

from torch import Tensor, empty, zeros
from torch.nn import Parameter

from ...simulator.configs import TorchInferenceRPUConfig
from ...simulator.parameters import (
    WeightClipType,
    WeightModifierType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
)

_LEGACY_NOISE = {
    WeightModifierType.ADD_NORMAL: WeightNoiseInjectionType.ADD_NORMAL,
    WeightModifierType.DISCRETIZE_ADD_NORMAL: WeightNoiseInjectionType.ADD_NORMAL,
    WeightModifierType.ADD_NORMAL_PER_CHANNEL: WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL,
    WeightModifierType.DISCRETIZE_ADD_NORMAL_PER_CHANNEL:
        WeightNoiseInjectionType.ADD_NORMAL_PER_CHANNEL,
}
_LEGACY_QUANT = {
    WeightModifierType.DISCRETIZE: WeightQuantizationType.DISCRETIZE,
    WeightModifierType.DISCRETIZE_ADD_NORMAL: WeightQuantizationType.DISCRETIZE,
    WeightModifierType.DISCRETIZE_PER_CHANNEL: WeightQuantizationType.DISCRETIZE_PER_CHANNEL,
    WeightModifierType.DISCRETIZE_ADD_NORMAL_PER_CHANNEL:
        WeightQuantizationType.DISCRETIZE_PER_CHANNEL,
}


class AnalogLayerBase:
    """Layer-level functionality common to analog modules."""

    # pylint: disable=no-member, attribute-defined-outside-init

    rpu_config: TorchInferenceRPUConfig
    in_sizes: List[int]
    register_buffer: Any

    IS_CONTAINER: bool = False
    """Containers (``AnalogSequential``, ``AnalogWrapper``) are skipped by the generators."""

    def named_analog_layers(self) -> Generator[Tuple[str, "AnalogLayerBase"], None, None]:
        """Yield ``(name, layer)`` for every non-container analog sub-module (self included)."""
        for name, layer in self.named_modules():  # type: ignore[attr-defined]
            if isinstance(layer, AnalogLayerBase) and not layer.IS_CONTAINER:
                yield name, layer

    def analog_layers(self) -> Generator["AnalogLayerBase", None, None]:
        """Yield every non-container analog sub-module."""
        for _, layer in self.named_analog_layers():
            yield layer

    def apply_to_analog_layers(self, fn: Callable) -> "AnalogLayerBase":
        """Call ``fn(layer)`` on every analog layer; returns self."""
        for layer in self.analog_layers():
            fn(layer)
        return self

    @classmethod
    def move_to_meta(cls, _):
        """Hook used by model conversion; nothing to do at this level."""
        return

    def clip_weights(self) -> None:
        """Clip the weights (overridden by layers that own weights)."""
        return

    def init_learnable_weight_ranges(self, init_value: Tensor, device, dtype) -> None:
        """Create ``learnable_weight_clip`` ``[T, N]`` when the clip type asks for it."""
        if self.rpu_config.clip.type == WeightClipType.LEARNABLE_PER_CHANNEL:
            self.learnable_weight_clip = Parameter(
                data=init_value.to(dtype=dtype, device=device), requires_grad=True
            )
        else:
            self.learnable_weight_clip = None  # type: ignore[assignment]

    def init_ir(self, device, dtype, init_value_ir: float, init_value_counter: int = 0) -> None:
        """Create the per-tile input-range state.

        Static (learned or calibrated) ranges: Parameter ``input_range [T]`` and the buffers
        ``input_range_update_idx``, ``x_min``, ``x_max`` ``[T]`` in the layer dtype. Disabled or
        dynamic ranges: all four are ``None``.
        """
        ir_config = self.rpu_config.pre_post.input_range
        n_tiles = len(self.in_sizes)
        if ir_config.enable and not ir_config.dynamic:
            self.input_range = Parameter(
                data=empty((n_tiles,), dtype=dtype, device=device).fill_(init_value_ir),
                requires_grad=ir_config.learn_input_range,
            )
            self.register_buffer(
                "input_range_update_idx",
                empty((n_tiles,), dtype=dtype, device=device).fill_(init_value_counter),
            )
            self.register_buffer("x_min", zeros((n_tiles,), dtype=dtype, device=device) - 1e-5)
            self.register_buffer("x_max", zeros((n_tiles,), dtype=dtype, device=device) + 1e-5)
        else:
            self.input_range = None  # type: ignore[assignment]
            self.input_range_update_idx = None
            self.x_min = None  # type: ignore[assignment]
            self.x_max = None  # type: ignore[assignment]

    def deprecation_adjustment(self) -> None:
        """Translate pre-v2 ``modifier.type`` / ``enable_during_test`` settings in place."""
        modifier = self.rpu_config.modifier
        if modifier.type != WeightModifierType.NONE:
            warnings.warn(
                "You are using the deprecated rpu_config.modifier.type. This model was likely "
                "trained with AIHWKIT-Lightning version <2."
            )
            modifier.noise_type = _LEGACY_NOISE.get(modifier.type, WeightNoiseInjectionType.NONE)
            modifier.quantization_type = _LEGACY_QUANT.get(
                modifier.type, WeightQuantizationType.NONE
            )
        if modifier.enable_during_test:
            modifier.enable_during_test = False
            warnings.warn(
                "You created a modifier with enable_during_test set True. "
                "This is deprecated and was set to False."
            )

    def quantize_weights(self) -> None:
        """After in-place quantisation the on-the-fly quantiser and clipping are switched off."""
        warnings.warn("Modified the rpu_config because quantize_weights was called.")
        self.rpu_config.modifier.quantization_type = WeightQuantizationType.NONE
        self.rpu_config.clip.type = WeightClipType.NONE

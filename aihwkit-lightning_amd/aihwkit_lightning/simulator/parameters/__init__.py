"""Parameter dataclasses and enums."""
from .enums import (
    WeightNoiseInjectionType,
    WeightQuantizationType,
    WeightClipType,
    WeightModifierType,
)
from .io import IOParameters
from .mapping import MappingParameter
from .pre_post import InputRangeParameter, PrePostProcessingParameter
from .inference import WeightModifierParameter, WeightClipParameter

__all__ = [
    "WeightNoiseInjectionType",
    "WeightQuantizationType",
    "WeightClipType",
    "WeightModifierType",
    "IOParameters",
    "MappingParameter",
    "InputRangeParameter",
    "PrePostProcessingParameter",
    "WeightModifierParameter",
    "WeightClipParameter",
]

"""Parameter dataclasses and enums."""
from .enums import (WeightClipType, WeightModifierType, WeightNoiseInjectionType,
                    WeightQuantizationType)
from .inference import WeightClipParameter, WeightModifierParameter
from .io import IOParameters
from .mapping import MappingParameter
from .pre_post import InputRangeParameter, PrePostProcessingParameter

__all__ = ["WeightNoiseInjectionType", "WeightQuantizationType", "WeightClipType",
           "WeightModifierType", "IOParameters", "MappingParameter", "InputRangeParameter",
           "PrePostProcessingParameter", "WeightModifierParameter", "WeightClipParameter"]

"""Public config namespace (same re-exports as reference ``simulator/configs/__init__.py``)."""
from ..parameters import (
    IOParameters,
    WeightModifierParameter,
    WeightClipParameter,
    MappingParameter,
    InputRangeParameter,
    PrePostProcessingParameter,
)
from ..parameters.enums import (
    WeightModifierType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
    WeightClipType,
)
from .configs import TorchInferenceRPUConfig

__all__ = [
    "IOParameters",
    "WeightModifierParameter",
    "WeightClipParameter",
    "MappingParameter",
    "InputRangeParameter",
    "PrePostProcessingParameter",
    "WeightModifierType",
    "WeightNoiseInjectionType",
    "WeightQuantizationType",
    "WeightClipType",
    "TorchInferenceRPUConfig",
]

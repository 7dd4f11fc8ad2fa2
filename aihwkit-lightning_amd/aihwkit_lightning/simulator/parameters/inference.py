"""Weight modifier and clip settings (reference ``inference.py:29-90``)."""
from dataclasses import dataclass, field
from .helpers import _PrintableMixin
from .enums import (
    WeightModifierType,
    WeightNoiseInjectionType,
    WeightQuantizationType,
    WeightClipType,
)


@dataclass
class WeightModifierParameter(_PrintableMixin):
    """Noise (``std_dev``, relative to max|W|) and quantisation (``res``) of the weights
    used in the training forward. ``type`` and ``enable_during_test`` are legacy fields."""

    std_dev: float = 0.0
    res: float = 0.0
    enable_during_test: bool = False
    type: WeightModifierType = field(
        default_factory=lambda: WeightModifierType.NONE, metadata={"always_show": True}
    )
    noise_type: WeightNoiseInjectionType = field(
        default_factory=lambda: WeightNoiseInjectionType.NONE, metadata={"always_show": True}
    )
    quantization_type: WeightQuantizationType = field(
        default_factory=lambda: WeightQuantizationType.NONE, metadata={"always_show": True}
    )


@dataclass
class WeightClipParameter(_PrintableMixin):
    """Clip bound ``sigma`` (in standard deviations); inactive while ``type`` is NONE."""

    sigma: float = -1.0
    type: WeightClipType = field(
        default_factory=lambda: WeightClipType.NONE, metadata={"always_show": True}
    )

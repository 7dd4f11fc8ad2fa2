"""Weight modifier and clip settings (reference ``inference.py:29-90``)."""
from dataclasses import dataclass

from . import enums
from .helpers import _PrintableMixin, shown


@dataclass
class WeightModifierParameter(_PrintableMixin):
    """Noise (``std_dev``, relative to max|W|) and quantisation (``res``: a number of states or
    its inverse) of the weights used in the training forward. ``type`` and
    ``enable_during_test`` are legacy fields kept for configs written for older versions."""

    std_dev: float = 0.0
    res: float = 0.0
    enable_during_test: bool = False
    type: enums.WeightModifierType = shown(enums.WeightModifierType.NONE)
    noise_type: enums.WeightNoiseInjectionType = shown(enums.WeightNoiseInjectionType.NONE)
    quantization_type: enums.WeightQuantizationType = shown(enums.WeightQuantizationType.NONE)


@dataclass
class WeightClipParameter(_PrintableMixin):
    """Clip bound ``sigma`` (in standard deviations); inactive while ``type`` is NONE."""

    sigma: float = -1.0
    type: enums.WeightClipType = shown(enums.WeightClipType.NONE)

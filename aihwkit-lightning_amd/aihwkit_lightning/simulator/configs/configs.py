"""The RPU configuration consumed by every analog layer (reference ``configs.py:27-88``)."""
from dataclasses import dataclass, field
from ..parameters import (
    IOParameters,
    WeightClipParameter,
    WeightModifierParameter,
    MappingParameter,
    PrePostProcessingParameter,
)


@dataclass
class TorchInferenceRPUConfig:
    """Hardware-aware-training configuration: forward non-idealities only, ideal backward.

    ``forward``  DAC/ADC resolution, output bound, output noise.
    ``clip``     weight clipping after optimizer steps / learned clipping.
    ``modifier`` weight noise and on-the-fly weight quantisation during training.
    ``mapping``  tile size along the input dimension.
    ``pre_post`` input-range handling.
    """

    forward: IOParameters = field(
        default_factory=IOParameters, metadata=dict(bindings_include=True)
    )
    clip: WeightClipParameter = field(default_factory=WeightClipParameter)
    modifier: WeightModifierParameter = field(default_factory=WeightModifierParameter)
    mapping: MappingParameter = field(default_factory=MappingParameter)
    pre_post: PrePostProcessingParameter = field(default_factory=PrePostProcessingParameter)

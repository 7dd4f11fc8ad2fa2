"""Digital pre/post-processing: the per-tile input range (reference ``pre_post.py:22-104``)."""
from dataclasses import dataclass, field
from .helpers import _PrintableMixin


@dataclass
class InputRangeParameter(_PrintableMixin):
    """Input range (DAC clipping bound) handling.

    ``enable`` off: no clipping (then no DAC quantisation either).
    ``dynamic``: range = abs-max of every input vector inside each tile.
    otherwise a learned per-tile scalar, initialised to ``init_value`` and, for the
    first ``init_from_data`` training batches, pulled towards ``init_std_alpha * std(x)``.
    Gradient: clipped inputs push the range out; ``decay`` pulls it in while more than
    ``input_min_percentage`` of the inputs are unclipped.
    """

    fast_mode: bool = False
    act_range_momentum: float = 0.95
    enable: bool = field(default_factory=lambda: False, metadata={"always_show": True})
    dynamic: bool = False
    learn_input_range: bool = True
    init_value: float = 3.0
    init_from_data: int = 100
    init_std_alpha: float = 3.0
    decay: float = 0.001
    input_min_percentage: float = 0.95


@dataclass
class PrePostProcessingParameter(_PrintableMixin):
    """Container for the input-range settings."""

    input_range: InputRangeParameter = field(default_factory=InputRangeParameter)


@dataclass
class PrePostProcessingRPU(_PrintableMixin):
    """Holder giving a config a ``pre_post`` member."""

    pre_post: PrePostProcessingParameter = field(default_factory=PrePostProcessingParameter)

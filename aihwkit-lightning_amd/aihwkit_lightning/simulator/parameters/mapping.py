"""Mapping of a logical weight matrix to physical tiles (reference ``mapping.py:21-46``)."""
from dataclasses import dataclass, field
from .helpers import _PrintableMixin


@dataclass
class MappingParameter(_PrintableMixin):
    """``max_input_size`` rows per analog tile along the input dimension; -1 = one tile."""

    max_input_size: int = -1


@dataclass
class MappableRPU(_PrintableMixin):
    """Holder giving a config a ``mapping`` member."""

    mapping: MappingParameter = field(default_factory=MappingParameter)

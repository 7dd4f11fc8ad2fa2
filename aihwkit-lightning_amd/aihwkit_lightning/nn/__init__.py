"""Analog neural-network modules (the AnalogLinear path)."""
from .modules.base import AnalogLayerBase
from .modules.container import AnalogSequential, AnalogWrapper
from .modules.linear import AnalogLinear
from .modules.hip_utils.hip_linear import HipLinear

__all__ = ["AnalogLayerBase", "AnalogSequential", "AnalogWrapper", "AnalogLinear", "HipLinear"]

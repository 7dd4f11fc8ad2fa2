"""Analog neural-network modules: AnalogLinear and the convolutions built on its operator."""
from .modules.base import AnalogLayerBase
from .modules.container import AnalogSequential, AnalogWrapper
from .modules.linear import AnalogLinear
from .modules.conv import AnalogConv1d, AnalogConv2d, AnalogConv3d
from .modules.hip_utils.hip_linear import HipLinear

__all__ = ["AnalogLayerBase", "AnalogSequential", "AnalogWrapper", "AnalogLinear", "AnalogConv1d",
           "AnalogConv2d", "AnalogConv3d", "HipLinear"]

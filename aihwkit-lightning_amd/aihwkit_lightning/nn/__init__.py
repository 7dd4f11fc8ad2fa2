"""Analog neural-network modules: AnalogLinear and the convolutions and recurrent layers built on
its operator."""
from .modules.base import AnalogLayerBase
from .modules.container import AnalogSequential, AnalogWrapper
from .modules.linear import AnalogLinear
from .modules.conv import AnalogConv1d, AnalogConv2d, AnalogConv3d
from .modules.rnn.rnn import AnalogRNN
from .modules.rnn.cells import (AnalogGRUCell, AnalogLSTMCell, AnalogLSTMCellCombinedWeight,
                                AnalogVanillaRNNCell)
from .modules.hip_utils.hip_linear import HipLinear

__all__ = ["AnalogLayerBase", "AnalogSequential", "AnalogWrapper", "AnalogLinear", "AnalogConv1d",
           "AnalogConv2d", "AnalogConv3d", "AnalogRNN", "AnalogVanillaRNNCell", "AnalogLSTMCell",
           "AnalogGRUCell", "AnalogLSTMCellCombinedWeight", "HipLinear"]

"""Enumerations selecting weight noise, quantisation and clipping behaviour.

Member names and string values follow reference ``simulator/parameters/enums.py:21-90``
because they are stored in checkpoints and user configs.
"""
from enum import Enum


class WeightModifierType(Enum):
    """Pre-v2 combined modifier selector; translated on layer construction."""

    NONE = "None"
    DISCRETIZE = "Discretize"
    DISCRETIZE_PER_CHANNEL = "DiscretizePerChannel"
    ADD_NORMAL = "AddNormal"
    ADD_NORMAL_PER_CHANNEL = "AddNormalPerChannel"
    DISCRETIZE_ADD_NORMAL = "DiscretizeAddNormal"
    DISCRETIZE_ADD_NORMAL_PER_CHANNEL = "DiscretizeAddNormalPerChannel"


class WeightNoiseInjectionType(Enum):
    """Gaussian weight noise drawn fresh in every training forward."""

    NONE = "None"
    ADD_NORMAL = "AddNormal"  # std = std_dev * max|W_tile|
    ADD_NORMAL_PER_CHANNEL = "AddNormalPerChannel"  # std = std_dev * max|W_tile[n, :]|


class WeightQuantizationType(Enum):
    """Uniform weight quantisation applied on the fly."""

    NONE = "None"
    DISCRETIZE = "Discretize"  # one scale per tile
    DISCRETIZE_PER_CHANNEL = "DiscretizePerChannel"  # one scale per tile and output channel


class WeightClipType(Enum):
    """Weight clipping after each optimizer step (or learned clipping in the forward)."""

    NONE = "None"
    LAYER_GAUSSIAN = "LayerGaussian"  # clamp at sigma * std(W)
    LAYER_GAUSSIAN_PER_CHANNEL = "LayerGaussianPerChannel"  # clamp at sigma * std(W[n, :])
    LEARNABLE_PER_CHANNEL = "LearnablePerChannel"  # LSQ-style learned per-channel range

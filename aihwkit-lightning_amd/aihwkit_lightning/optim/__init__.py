"""Optimizers for hardware-aware training."""
from .analog_optimizer import AnalogOptimizer

__all__ = ["AnalogOptimizer"]

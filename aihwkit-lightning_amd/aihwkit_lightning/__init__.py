"""MI355X-native drop-in for the AnalogLinear hot path of aihwkit-lightning.

The package keeps the reference's import paths (``aihwkit_lightning.nn``,
``aihwkit_lightning.simulator.configs``, ``aihwkit_lightning.optim``,
``aihwkit_lightning.inference``) but every arithmetic operation of the layer
runs in hand-written HIP kernels for gfx950 behind a C-ABI shared library.
There is no CPU or eager-PyTorch compute fallback.
"""
from .version import __version__

__all__ = ["__version__"]

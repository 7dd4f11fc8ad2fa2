"""Public config namespace (same re-exports as reference ``simulator/configs/__init__.py``)."""
from .. import parameters as _p
from ..parameters import *  # noqa: F401,F403  (the names listed in parameters.__all__)
from .configs import TorchInferenceRPUConfig

__all__ = [*_p.__all__, "TorchInferenceRPUConfig"]

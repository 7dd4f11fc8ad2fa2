"""Exception hierarchy (same names as reference ``exceptions.py:16-33``)."""


class AihwkitException(Exception):
    """Root of all errors raised by this package."""


class ModuleError(AihwkitException):
    """A problem with an analog module (shape, state, device)."""


class ArgumentError(AihwkitException):
    """A call received arguments it cannot work with."""


class ConfigError(AihwkitException):
    """The RPU configuration asks for something unsupported or inconsistent."""


class TorchTileConfigError(ConfigError):
    """Configuration error specific to a tile implementation."""


class HipBackendError(AihwkitException):
    """The HIP library is missing, failed to load, or a kernel launch was rejected."""

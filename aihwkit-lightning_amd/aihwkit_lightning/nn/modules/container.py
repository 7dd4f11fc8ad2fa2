"""Containers that propagate analog-layer operations (reference ``nn/modules/container.py``)."""
from collections import OrderedDict
from types import new_class
from typing import Any, Dict, Optional, Type

from torch.nn import Module, Sequential

from .base import AnalogLayerBase


class AnalogContainerBase(AnalogLayerBase):
    """Marks a module as a container: it is skipped by ``analog_layers()``."""

    IS_CONTAINER: bool = True


class AnalogSequential(AnalogContainerBase, Sequential):
    """``nn.Sequential`` with the analog-layer mixin."""

    # pylint: disable=unused-argument
    @classmethod
    def from_digital(cls, module: Sequential, *args: Any, **kwargs: Any) -> "AnalogSequential":
        """Re-wrap the children of a ``Sequential``."""
        return cls(OrderedDict(module.named_children()))

    @classmethod
    def to_digital(cls, module: "AnalogSequential", *args: Any, **kwargs: Any) -> Sequential:
        """Back to a plain ``Sequential`` over the same children."""
        return Sequential(OrderedDict(module.named_children()))


class AnalogWrapper(AnalogContainerBase):
    """Adds the analog-layer mixin to an arbitrary module by dynamic subclassing; the wrapped
    module's state is shared, not copied."""

    SUBCLASSES: Dict[str, Type] = {}

    def __new__(cls, module: Optional[Module] = None, **__: Any) -> "AnalogWrapper":
        if module is None:  # deepcopy / pickle
            return super().__new__(cls)
        name = f"{cls.__name__}{type(module).__name__}"
        if name not in cls.SUBCLASSES:
            cls.SUBCLASSES[name] = new_class(name, (cls, type(module)), {})
        return super().__new__(cls.SUBCLASSES[name])

    def __init__(self, module: Module):  # pylint: disable=super-init-not-called
        self.__dict__.update(module.__dict__)

    @classmethod
    def _rebuild(cls, wrapped_class: Type) -> "AnalogWrapper":
        """An empty instance of the wrapper class of ``wrapped_class`` (for unpickling)."""
        return cls.__new__(cls, wrapped_class.__new__(wrapped_class))

    def __reduce__(self):
        # the dynamic class cannot be looked up by name: pickle the wrapped class (which can)
        # and the state, and build the wrapper class again when loading
        return (AnalogWrapper._rebuild, (type(self).__bases__[1],), self.__dict__)

    # pylint: disable=unused-argument
    @classmethod
    def from_digital(cls, module: Module, *args: Any, **kwargs: Any) -> "AnalogWrapper":
        """Wrap ``module``."""
        return cls(module)

    @classmethod
    def to_digital(cls, module: "AnalogWrapper", *args: Any, **kwargs: Any) -> Module:
        """Unwrap: an instance of the original class sharing the same state."""
        digital_class = type(module).__bases__[1]
        plain = digital_class.__new__(digital_class)  # type: ignore[call-overload]
        plain.__dict__ = module.__dict__
        return plain

    def quantize_weights(self) -> None:
        """Quantise the weights of every analog layer in place."""
        for layer in self.analog_layers():
            layer.quantize_weights()

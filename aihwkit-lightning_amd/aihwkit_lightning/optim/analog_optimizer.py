"""``AnalogOptimizer``: any torch optimizer plus weight clipping after each step
(reference ``optim/analog_optimizer.py:23-79``)."""
from types import new_class
from typing import Any, Callable, Dict, Generator, Type

from torch.optim import Optimizer


class AnalogOptimizer(Optimizer):
    """``AnalogOptimizer(OptCls, analog_layers_callable, params, **kwargs)`` returns an instance
    of a class deriving from both ``AnalogOptimizer`` and ``OptCls``. After every ``step()`` a
    post hook calls ``clip_weights()`` on each layer yielded by ``analog_layers_callable()``.
    """

    SUBCLASSES: Dict[str, Type] = {}

    def __new__(cls, optimizer_cls: Type, *_: Any, **__: Any) -> "AnalogOptimizer":
        name = f"{cls.__name__}{optimizer_cls.__name__}"
        if name not in cls.SUBCLASSES:
            cls.SUBCLASSES[name] = new_class(name, (cls, optimizer_cls), {})
        return super().__new__(cls.SUBCLASSES[name])

    def __init__(self, _: Type, analog_layers: Callable[[], Generator], *args: Any, **kwargs: Any):
        super().__init__(*args, **kwargs)

        def clip_after_step(*_args: Any, **_kwargs: Any) -> None:
            for layer in analog_layers():
                layer.clip_weights()

        self.register_step_post_hook(clip_after_step)

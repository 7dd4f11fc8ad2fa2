"""Swap the digital layers of a model for their analog counterparts and back (reference
``nn/conversion.py:37-300``): ``Linear`` and ``Conv1d/2d/3d`` map onto the layers built on the HIP
operator, ``Sequential`` onto ``AnalogSequential``, ``RNN`` / ``LSTM`` / ``GRU`` onto ``AnalogRNN``."""
from copy import deepcopy
from typing import Callable, Dict, List, Optional, Set, Union

from torch.nn import GRU, LSTM, RNN, Conv1d, Conv2d, Conv3d, Linear, Module, Sequential

from ..exceptions import ArgumentError
from ..simulator.configs import TorchInferenceRPUConfig
from .modules.base import AnalogLayerBase
from .modules.container import AnalogSequential, AnalogWrapper
from .modules.conv import AnalogConv1d, AnalogConv2d, AnalogConv3d
from .modules.linear import AnalogLinear
from .modules.rnn.rnn import AnalogRNN

_DEFAULT_CONVERSION_MAP = {
    Linear: AnalogLinear,
    Conv1d: AnalogConv1d,
    Conv2d: AnalogConv2d,
    Conv3d: AnalogConv3d,
    Sequential: AnalogSequential,
    LSTM: AnalogRNN,
    GRU: AnalogRNN,
    RNN: AnalogRNN,
}
_DEFAULT_DIGITAL_CONVERSION_SET = {*_DEFAULT_CONVERSION_MAP.values()}


def specific_rpu_config_id(
    module_name: str, module: Module, rpu_config: TorchInferenceRPUConfig
) -> TorchInferenceRPUConfig:
    """Default per-layer hook: every layer gets the generic config unchanged."""
    # pylint: disable=unused-argument
    return rpu_config


def _join(parent: str, child: str) -> str:
    return f"{parent}.{child}" if parent else child


def convert_to_analog(
    module: Module,
    rpu_config: TorchInferenceRPUConfig,
    conversion_map: Optional[Dict] = None,
    specific_rpu_config_fun: Optional[Callable] = None,
    module_name: str = "",
    ensure_analog_root: bool = True,
    exclude_modules: Optional[List[str]] = None,
    inplace: bool = False,
    verbose: bool = False,
) -> Union[Module, AnalogWrapper]:
    """Return ``module`` with every layer whose class is a key of ``conversion_map`` replaced by
    ``conversion_map[cls].from_digital(layer, config)``; each layer gets its own deep copy of
    ``rpu_config``, passed through ``specific_rpu_config_fun(name, layer, config)``. Names in
    ``exclude_modules`` are left alone. Without ``inplace`` the model is deep-copied first; with
    it, converted digital layers release their storage. A root that is not itself an analog
    layer is wrapped in ``AnalogWrapper`` unless ``ensure_analog_root`` is off."""
    # pylint: disable=too-many-arguments
    exclude = list(exclude_modules or [])
    if conversion_map is None:
        conversion_map = _DEFAULT_CONVERSION_MAP
    if not isinstance(conversion_map, dict):
        raise ArgumentError("Conversion map should be a dictionary")
    config_fun = specific_rpu_config_fun or specific_rpu_config_id
    if not inplace:
        module = deepcopy(module)

    def to_analog(name: str, layer: Module) -> Module:
        analog_cls = conversion_map[layer.__class__]
        converted = analog_cls.from_digital(layer, config_fun(name, layer, deepcopy(rpu_config)))
        if verbose:
            print(f"Converted '{name}' to '{analog_cls.__name__}'.")
        return converted

    def walk(name: str, layer: Module) -> Module:
        if layer.__class__ in conversion_map and name not in exclude:
            converted = to_analog(name, layer)
            if inplace and name == module_name:
                conversion_map[layer.__class__].move_to_meta(layer)
            layer = converted
        replaced = {}
        for child_name, child in layer.named_children():
            full = _join(name, child_name)
            if full in exclude:
                continue
            if any(True for _ in child.named_children()):
                replaced[child_name] = walk(full, child)
            elif child.__class__ in conversion_map:
                replaced[child_name] = to_analog(full, child)
        for child_name, new_child in replaced.items():
            layer._modules[child_name] = new_child  # pylint: disable=protected-access
        return layer

    root = walk(module_name, module)
    if ensure_analog_root and not module_name and not isinstance(root, AnalogLayerBase):
        return AnalogWrapper(root)
    return root


def convert_to_digital(
    module: Module,
    conversion_set: Optional[Set] = None,
    module_name: str = "",
    inplace: bool = False,
) -> Module:
    """Inverse of :func:`convert_to_analog`: every layer whose class is in ``conversion_set`` (by
    default all analog layers of this package) and every ``AnalogWrapper`` is replaced by
    ``cls.to_digital(layer)``."""
    if conversion_set is None:
        conversion_set = _DEFAULT_DIGITAL_CONVERSION_SET
    if not isinstance(conversion_set, set):
        raise ArgumentError("Conversion set should be a set")
    if not inplace:
        module = deepcopy(module)

    def to_digital(layer: Module) -> Module:
        if not hasattr(layer.__class__, "to_digital"):
            raise ArgumentError(
                "The conversion set should only contain analog layers that support "
                "`to_digital` conversion."
            )
        return layer.__class__.to_digital(layer)

    def walk(name: str, layer: Module) -> Module:
        if layer.__class__ in conversion_set or isinstance(layer, AnalogWrapper):
            layer = to_digital(layer)
        replaced = {}
        for child_name, child in layer.named_children():
            if any(True for _ in child.named_children()):
                replaced[child_name] = walk(_join(name, child_name), child)
            elif child.__class__ in conversion_set:
                replaced[child_name] = to_digital(child)
        for child_name, new_child in replaced.items():
            layer._modules[child_name] = new_child  # pylint: disable=protected-access
        return layer

    return walk(module_name, module)

"""``AnalogRNN``: stacked (optionally bidirectional) recurrent layers on analog tiles, the analog
counterpart of ``torch.nn.RNN`` / ``LSTM`` / ``GRU`` (reference ``nn/modules/rnn/rnn.py:41-642``).

The module tree (``rnn.layers[i](.directions[d]).cell.weight_ih|weight_hh``) is the reference's,
so checkpoints of the module tree are interchangeable; the state dict itself is exposed in
torch's flat naming (``weight_ih_l0``, ``bias_hh_l1_reverse``, ``input_range_ih_l0`` ...), as the
reference does, and both namings are accepted on load.
"""
import math
import re
import warnings
from typing import Any, Callable, Dict, Iterator, List, Optional, Tuple, Type, Union

import torch
from torch import Tensor
from torch.nn import GRU, LSTM, RNN, Dropout, Linear, Module, ModuleList, init

from ..container import AnalogContainerBase
from ..linear import AnalogLinear
from .cells import AnalogGRUCell, AnalogLSTMCell, AnalogVanillaRNNCell, LSTMState
from .layers import AnalogBidirRNNLayer, AnalogRNNLayer
from ....simulator.configs import TorchInferenceRPUConfig

_FLAT_KEY = re.compile(r"^(?P<tensor>\w+?)_(?P<part>ih|hh)_l(?P<layer>\d+)(?P<rev>_reverse)?$")
_TREE_KEY = re.compile(
    r"^rnn\.layers\.(?P<layer>\d+)\.(?:directions\.(?P<dir>\d)\.)?cell\.weight_(?P<part>ih|hh)"
    r"\.(?P<tensor>\w+)$"
)
_CELL_OF = {RNN: AnalogVanillaRNNCell, LSTM: AnalogLSTMCell, GRU: AnalogGRUCell}


class ModularRNN(Module):
    """``num_layers`` recurrent layers in series with dropout between them (reference
    rnn.py:41-138). ``first_layer_args`` / ``other_layer_args`` are the constructor arguments of
    ``layer`` for the first and the remaining layers."""

    def __init__(
        self,
        num_layers: int,
        layer: Union[Type[AnalogBidirRNNLayer], Type[AnalogRNNLayer]],
        dropout: float,
        first_layer_args: Any,
        other_layer_args: Any,
    ) -> None:
        super().__init__()
        self.layers = ModuleList(
            [layer(*(first_layer_args if i == 0 else other_layer_args)) for i in range(num_layers)]
        )
        self.num_layers = num_layers
        if num_layers == 1 and dropout > 0:
            warnings.warn(
                "dropout is applied between recurrent layers and has no effect with "
                "num_layers = 1"
            )
        self.dropout_layer = Dropout(dropout) if dropout > 0.0 else None

    def get_zero_state(self, batch_size: int) -> List:
        """One all-zero state per layer."""
        return [layer.get_zero_state(batch_size) for layer in self.layers]

    def forward(self, inp: Tensor, states: List) -> Tuple[Tensor, List]:
        """``inp [steps, batch, features]`` through all layers: (output, last state per layer)."""
        last_states = []
        for i, (layer, state) in enumerate(zip(self.layers, states)):
            inp, last = layer(inp, state)
            if self.dropout_layer is not None and i + 1 < self.num_layers:
                inp = self.dropout_layer(inp)
            last_states.append(last)
        return inp, last_states


class GraphedRNN:
    """``net(inp, states)`` in evaluation mode for one input shape, recorded once as a HIP graph
    and replayed per call. A recurrent step is a handful of small launches (two analog products,
    ten element-wise kernels), so an eager sequence is bound by the host's launch rate; the graph
    removes the host from the loop. Nothing in the analog operator allocates, synchronises or
    clears memory outside kernels, so every launch of the sequence is recorded as a kernel node.

    The graph reads the parameters where they were when it was recorded: in-place updates are
    seen by later calls, re-assigned parameter tensors are not (record a new graph then). Calls
    return copies, so results survive the next call.
    """

    def __init__(self, net: "AnalogRNN", example_inp: Tensor, states: Optional[List] = None):
        if net.training:
            raise RuntimeError("GraphedRNN records the evaluation-mode forward; call net.eval()")
        if not example_inp.is_cuda:
            raise RuntimeError("GraphedRNN needs an input on the GPU")
        self.net = net
        self.inp = example_inp.detach().clone()
        batch = self.inp.size(1) if self.inp.dim() == 3 else 1
        self.states = self._clone_states(states if states is not None
                                         else net.get_zero_state(batch))
        self.given_states = states is not None
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.no_grad(), torch.cuda.stream(side):
            net(self.inp, self.states)  # loads the library and fills the host-side caches
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.no_grad(), torch.cuda.graph(self.graph):
            self.out, self.last = net(self.inp, self.states)

    @staticmethod
    def _map_states(fn, states):
        """``fn`` applied to every tensor of a nested list / tuple / ``LSTMState`` structure."""
        if states is None:
            return None
        if isinstance(states, Tensor):
            return fn(states)
        mapped = [GraphedRNN._map_states(fn, s) for s in states]
        if hasattr(states, "_fields"):
            return type(states)(*mapped)
        return type(states)(mapped)

    @classmethod
    def _clone_states(cls, states):
        return cls._map_states(lambda t: t.detach().clone(), states)

    def __call__(self, inp: Tensor, states: Optional[List] = None) -> Tuple[Tensor, List]:
        if inp.shape != self.inp.shape or inp.dtype != self.inp.dtype:
            raise RuntimeError(
                f"recorded for input {tuple(self.inp.shape)} {self.inp.dtype}, "
                f"got {tuple(inp.shape)} {inp.dtype}"
            )
        if (states is not None) != self.given_states:
            raise RuntimeError("recorded with" + ("" if self.given_states else "out")
                               + " initial states; call it the same way")
        self.inp.copy_(inp)
        if states is not None:
            flat_new, flat_own = [], []
            self._map_states(lambda t: flat_new.append(t) or t, states)
            self._map_states(lambda t: flat_own.append(t) or t, self.states)
            for own, new in zip(flat_own, flat_new):
                own.copy_(new)
        self.graph.replay()
        return self.out.clone(), self._map_states(lambda t: t.clone(), self.last)


class AnalogRNN(AnalogContainerBase, Module):
    """Recurrent network of ``cell`` (``AnalogVanillaRNNCell``, ``AnalogLSTMCell``,
    ``AnalogGRUCell`` or ``AnalogLSTMCellCombinedWeight``) with time-major input.

    ``forward(inp, states=None)`` takes ``inp [steps, batch, input_size]`` (or ``[steps,
    input_size]`` for one sequence) and one state per layer (a pair of states per layer when
    bidirectional) and returns the outputs of the last layer and the last states.
    ``batch_first`` and ``proj_size`` are not supported, as in the reference.
    """

    def __init__(
        self,
        cell: Type,
        input_size: int,
        hidden_size: int,
        num_layers: int = 1,
        bias: bool = True,
        batch_first: bool = False,
        bidir: bool = False,
        dropout: float = 0.0,
        proj_size: int = 0,
        xavier: bool = False,
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):  # pylint: disable=too-many-arguments
        super().__init__()
        if batch_first:
            raise RuntimeError("batch_first is not supported for AnalogRNN")
        if proj_size != 0:
            raise RuntimeError("proj_size != 0 not supported for AnalogRNN")
        fan_out = 2 * hidden_size if bidir else hidden_size
        tail = [hidden_size, bias, device, dtype, rpu_config]
        self.rnn = ModularRNN(
            num_layers,
            AnalogBidirRNNLayer if bidir else AnalogRNNLayer,
            dropout,
            first_layer_args=[cell, input_size, *tail],
            other_layer_args=[cell, fan_out, *tail],
        )
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.num_layers = num_layers
        self.batch_first = batch_first
        self.dropout = dropout
        self.bidirectional = bidir
        self.proj_size = 0
        self.reset_parameters(xavier)
        self._register_load_state_dict_pre_hook(self._accept_flat_keys)
        self._register_state_dict_hook(self._emit_flat_keys)

    # ------------------------------------------------------------------ initialisation
    @torch.no_grad()
    def init_layers(self, weight_init_fn: Callable, bias_init_fn: Optional[Callable] = None) -> None:
        """Apply the in-place initialisers to every projection (the weight initialiser also to
        the biases if no other is given)."""
        bias_init_fn = bias_init_fn or weight_init_fn
        for module in self.modules():
            if isinstance(module, AnalogLinear):
                weight, bias = module.get_weights_and_biases()
                weight_init_fn(weight.data)
                if bias is not None:
                    bias_init_fn(bias.data)
                module.set_weights_and_biases(weight, bias)
            elif isinstance(module, Linear):
                weight_init_fn(module.weight.data)
                if module.bias is not None:
                    bias_init_fn(module.bias.data)

    def reset_parameters(self, xavier: bool = False) -> None:
        """Uniform in ``+-1/sqrt(hidden_size)`` like torch's recurrent layers, or Xavier-uniform
        weights with zero biases."""
        if xavier:
            self.init_layers(init.xavier_uniform_, init.zeros_)
        else:
            bound = 1.0 / math.sqrt(self.hidden_size)
            self.init_layers(lambda t: t.uniform_(-bound, bound))

    # ------------------------------------------------------------------ forward
    def get_zero_state(self, batch_size: int) -> List:
        """All-zero initial states in the structure ``forward`` expects."""
        return self.rnn.get_zero_state(batch_size)

    def _flat(self, states: List) -> List[LSTMState]:
        return [s for pair in states for s in pair] if self.bidirectional else list(states)

    def forward(self, inp: Tensor, states: Optional[List] = None) -> Tuple[Tensor, List]:
        """Run the network; see the class docstring for shapes."""
        if inp.dim() not in (2, 3):
            raise RuntimeError(
                f"RNN: Expected input to be 2D or 3D, got {inp.dim()}D tensor instead"
            )
        if states is not None and len(states) != self.num_layers:
            raise RuntimeError(f"Expecting {self.num_layers} states, but received {len(states)}")
        batched = inp.dim() == 3
        if states is not None:
            want = 2 if batched else 1
            kind = "batched 3-D" if batched else "unbatched 2-D"
            for state in self._flat(states):
                for name in ("hx", "cx"):
                    tensor = getattr(state, name)
                    if tensor is None:  # cells without a cell state
                        continue
                    got = tensor.dim()
                    if got != want:
                        raise RuntimeError(
                            f"For {kind} input, {name} should be {want}-D but got {got}-D tensor"
                        )
        if not batched:
            inp = inp.unsqueeze(1)
        batch = inp.size(1)
        if states is None:
            states = self.get_zero_state(batch)
        for state in self._flat(states):
            self.check_forward_args(inp, state, batch)
        return self.rnn(inp, states)

    def check_input(self, inp: Tensor) -> None:
        """The feature dimension must be ``input_size``."""
        if self.input_size != inp.size(-1):
            raise RuntimeError(
                f"input.size(-1) must be equal to input_size. "
                f"Expected {self.input_size}, got {inp.size(-1)}"
            )

    def check_hidden_size(
        self, h_x: Tensor, expected_hidden_size: Tuple[int, int],
        msg: str = "Expected hidden size {}, got {}",
    ) -> None:
        """A state tensor must be ``[batch, hidden_size]``."""
        if tuple(h_x.size()) != tuple(expected_hidden_size):
            raise RuntimeError(msg.format(expected_hidden_size, list(h_x.size())))

    def check_forward_args(self, inp: Tensor, hidden: LSTMState, batch_size: int) -> None:
        """Shape checks of the input and one state."""
        self.check_input(inp)
        self.check_hidden_size(hidden.hx, (batch_size, self.hidden_size))
        if hidden.cx is not None:
            self.check_hidden_size(hidden.cx, (batch_size, self.hidden_size))

    def graphed(self, example_inp: Tensor, states: Optional[List] = None) -> GraphedRNN:
        """A callable with the signature of ``forward`` that replays the evaluation-mode forward
        for inputs of ``example_inp``'s shape as one HIP graph (see :class:`GraphedRNN`)."""
        return GraphedRNN(self, example_inp, states)

    # ------------------------------------------------------------------ cells and state dicts
    def cells(self) -> Iterator[Tuple[int, bool, Module]]:
        """``(layer index, is the reversed direction, cell)`` for every cell."""
        for i, layer in enumerate(self.rnn.layers):
            if self.bidirectional:
                yield i, False, layer.directions[0].cell
                yield i, True, layer.directions[1].cell
            else:
                yield i, False, layer.cell

    def _accept_flat_keys(self, state_dict: Dict, prefix: str, *_: Any) -> None:
        """Before loading: rename entries in torch's flat naming to the module tree's."""
        for key in [k for k in state_dict if k.startswith(prefix)]:
            found = _FLAT_KEY.match(key[len(prefix):])
            if found is None:
                continue
            where = f"rnn.layers.{found['layer']}."
            if self.bidirectional:
                where += f"directions.{1 if found['rev'] else 0}."
            state_dict[f"{prefix}{where}cell.weight_{found['part']}.{found['tensor']}"] = \
                state_dict.pop(key)

    @staticmethod
    def _emit_flat_keys(module: Module, state_dict: Dict, prefix: str, *_: Any) -> None:
        """After collecting: rename the module tree's entries to torch's flat naming."""
        # pylint: disable=unused-argument
        for key in [k for k in state_dict if k.startswith(prefix)]:
            found = _TREE_KEY.match(key[len(prefix):])
            if found is None:
                continue
            rev = "_reverse" if found["dir"] == "1" else ""
            flat = f"{found['tensor']}_{found['part']}_l{found['layer']}{rev}"
            state_dict[prefix + flat] = state_dict.pop(key)

    # ------------------------------------------------------------------ conversion
    @classmethod
    def from_digital(
        cls,
        module: Union[RNN, LSTM, GRU],
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
        realistic_read_write: bool = False,
    ) -> "AnalogRNN":
        """Analog network with the structure and weights of a torch ``RNN`` / ``LSTM`` / ``GRU``
        (the third argument is passed on as the constructor's ``xavier`` flag, as in the
        reference; the initial values it selects are overwritten by the copied weights)."""
        analog = cls(
            _CELL_OF[type(module)], module.input_size, module.hidden_size, module.num_layers,
            module.bias is not False, module.batch_first, module.bidirectional, module.dropout,
            module.proj_size, realistic_read_write, module.weight_hh_l0.device,
            module.weight_hh_l0.dtype, rpu_config,
        )
        for layer, reverse, cell in analog.cells():
            tag = f"l{layer}" + ("_reverse" if reverse else "")
            for part in ("ih", "hh"):
                bias = getattr(module, f"bias_{part}_{tag}") if module.bias is not False else None
                getattr(cell, f"weight_{part}").set_weights_and_biases(
                    getattr(module, f"weight_{part}_{tag}"), bias
                )
        return analog

    @classmethod
    def to_digital(cls, module: "AnalogRNN") -> Union[RNN, LSTM, GRU]:
        """torch ``RNN`` (tanh) / ``LSTM`` / ``GRU`` with the same structure and weights."""
        _, _, first = next(module.cells())
        proj = first.weight_ih
        device, dtype = proj.weight.device, proj.weight.dtype
        has_bias = proj.bias is not None
        common = dict(
            num_layers=module.num_layers, bias=has_bias, batch_first=module.batch_first,
            dropout=module.dropout, bidirectional=module.bidirectional, device=device, dtype=dtype,
        )
        if isinstance(first, AnalogVanillaRNNCell):
            digital = RNN(module.input_size, module.hidden_size, nonlinearity="tanh", **common)
        elif isinstance(first, AnalogLSTMCell):
            digital = LSTM(module.input_size, module.hidden_size, proj_size=module.proj_size,
                           **common)
        elif isinstance(first, AnalogGRUCell):
            digital = GRU(module.input_size, module.hidden_size, **common)
        else:
            raise TypeError(f"no torch counterpart for cell type {type(first).__name__}")
        with torch.no_grad():
            for layer, reverse, cell in module.cells():
                tag = f"l{layer}" + ("_reverse" if reverse else "")
                for part in ("ih", "hh"):
                    proj = getattr(cell, f"weight_{part}")
                    getattr(digital, f"weight_{part}_{tag}").copy_(proj.weight.data)
                    if has_bias:
                        getattr(digital, f"bias_{part}_{tag}").copy_(proj.bias.data)
        return digital.to(device=device, dtype=dtype)

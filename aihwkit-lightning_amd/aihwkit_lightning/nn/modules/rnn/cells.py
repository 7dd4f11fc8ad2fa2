"""Recurrent cells whose matrix products run on analog tiles.

Same cells, parameters and arithmetic as the reference's ``nn/modules/rnn/cells.py:45-343``: each
cell owns ``AnalogLinear`` projections (``weight_ih`` for the input, ``weight_hh`` for the hidden
state, or one ``weight`` over their concatenation) and combines their outputs with the usual
element-wise gate formulas. A cell is split into ``project_input`` (the product that does not
depend on the recurrence) and ``recur`` (everything that does), so that a layer may compute the
input projection of a whole sequence in one product over ``steps * batch`` rows.
"""
from collections import namedtuple
from typing import Optional, Tuple

import torch
from torch import Tensor
from torch.nn import Module

from ..linear import AnalogLinear
from ....simulator.configs import TorchInferenceRPUConfig

LSTMState = namedtuple("LSTMState", ["hx", "cx"])


def lstm_pointwise(gates: Tensor, c_x: Tensor) -> Tuple[Tensor, Tensor]:
    """``(h_y, c_y)`` from the summed pre-activations ``[B, 4H]`` in the order input, forget,
    cell, output (reference cells.py:176-186)."""
    in_gate, forget_gate, cell_gate, out_gate = gates.chunk(4, 1)
    c_y = torch.sigmoid(forget_gate) * c_x + torch.sigmoid(in_gate) * torch.tanh(cell_gate)
    return torch.sigmoid(out_gate) * torch.tanh(c_y), c_y


class _AnalogCell(Module):
    """Common part of the cells with separate input and hidden projections: ``gate_count * H``
    output channels each."""

    gate_count = 1
    has_cell_state = False

    def __init__(
        self,
        input_size: int,
        hidden_size: int,
        bias: bool,
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        width = self.gate_count * hidden_size
        self.weight_ih = AnalogLinear(input_size, width, bias, device, dtype, rpu_config)
        self.weight_hh = AnalogLinear(hidden_size, width, bias, device, dtype, rpu_config)

    def get_zero_state(self, batch_size: int) -> LSTMState:
        """All-zero state for ``batch_size`` sequences; ``cx`` is None for cells without one."""
        like = next(self.parameters())
        zero = torch.zeros(batch_size, self.hidden_size, device=like.device, dtype=like.dtype)
        return LSTMState(zero, torch.zeros_like(zero) if self.has_cell_state else None)

    #: rows of a sequence are independent of the recurrence in ``project_input``
    input_projection_is_separate = True

    def project_input(self, input_: Tensor) -> Tensor:
        """Input part of the pre-activations, ``[rows, gate_count * H]``."""
        return self.weight_ih(input_)

    def recur(self, igates: Tensor, state) -> Tuple[Tensor, Tuple[Tensor, Optional[Tensor]]]:
        """One time step from the projected input and the previous state."""
        raise NotImplementedError

    def forward(self, input_: Tensor, state) -> Tuple[Tensor, Tuple[Tensor, Optional[Tensor]]]:
        """One time step: ``(output [B, H], (hx, cx or None))``."""
        return self.recur(self.project_input(input_), state)


class AnalogVanillaRNNCell(_AnalogCell):
    """``h' = tanh(W_ih x + W_hh h)`` (reference cells.py:45-113)."""

    gate_count = 1

    def recur(self, igates, state):
        h_x, _ = state
        out = torch.tanh(igates + self.weight_hh(h_x))
        return out, (out, None)


class AnalogLSTMCell(_AnalogCell):
    """LSTM cell, gates stacked as input, forget, cell, output (reference cells.py:116-191)."""

    gate_count = 4
    has_cell_state = True

    def recur(self, igates, state):
        h_x, c_x = state
        h_y, c_y = lstm_pointwise(igates + self.weight_hh(h_x), c_x)
        return h_y, (h_y, c_y)


class AnalogGRUCell(_AnalogCell):
    """GRU cell, gates stacked as reset, update, new; the reset gate scales the hidden part of
    the candidate after the product, as in ``torch.nn.GRU`` (reference cells.py:270-343)."""

    gate_count = 3

    def recur(self, igates, state):
        h_x, _ = state
        i_r, i_z, i_n = igates.chunk(3, 1)
        h_r, h_z, h_n = self.weight_hh(h_x).chunk(3, 1)
        reset = torch.sigmoid(i_r + h_r)
        update = torch.sigmoid(i_z + h_z)
        cand = torch.tanh(i_n + reset * h_n)
        h_y = cand + update * (h_x - cand)
        return h_y, (h_y, None)


class AnalogLSTMCellCombinedWeight(Module):
    """LSTM cell with one projection ``weight`` over ``[x, h]`` (reference cells.py:194-267): the
    input and hidden parts share tiles, so nothing can be projected ahead of the recurrence."""

    input_projection_is_separate = False

    def __init__(
        self,
        input_size: int,
        hidden_size: int,
        bias: bool,
        device=None,
        dtype=None,
        rpu_config: Optional[TorchInferenceRPUConfig] = None,
    ):
        super().__init__()
        self.input_size = input_size
        self.hidden_size = hidden_size
        self.weight = AnalogLinear(
            input_size + hidden_size, 4 * hidden_size, bias, device, dtype, rpu_config
        )

    def get_zero_state(self, batch_size: int) -> LSTMState:
        """All-zero hidden and cell state."""
        like = next(self.parameters())
        zero = torch.zeros(batch_size, self.hidden_size, device=like.device, dtype=like.dtype)
        return LSTMState(zero, torch.zeros_like(zero))

    def forward(self, input_: Tensor, state) -> Tuple[Tensor, Tuple[Tensor, Tensor]]:
        """One time step."""
        h_x, c_x = state
        h_y, c_y = lstm_pointwise(self.weight(torch.cat((input_, h_x), 1)), c_x)
        return h_y, (h_y, c_y)

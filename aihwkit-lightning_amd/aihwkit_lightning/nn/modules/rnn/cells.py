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
from torch.autograd import Function
from torch.nn import Module

from ..hip_utils import ops as gate_ops
from ..linear import AnalogLinear
from ....simulator.configs import TorchInferenceRPUConfig

LSTMState = namedtuple("LSTMState", ["hx", "cx"])


class _LstmGates(Function):
    """LSTM gate arithmetic of one step as one kernel per pass."""

    # pylint: disable=abstract-method, arguments-differ

    @staticmethod
    def forward(ctx, igates: Tensor, hgates: Optional[Tensor], c_x: Tensor):
        needs = any(ctx.needs_input_grad)
        c_x = gate_ops.dense(c_x)  # the backward pass reads it again
        h_y, c_y, act = gate_ops.lstm_gates_fwd(igates, hgates, c_x, needs)
        if needs:
            ctx.save_for_backward(act, c_x, c_y)
        ctx.two_products = hgates is not None
        ctx.set_materialize_grads(False)
        return h_y, c_y

    @staticmethod
    def backward(ctx, dh_y: Optional[Tensor], dc_y: Optional[Tensor]):
        act, c_x, c_y = ctx.saved_tensors
        if dh_y is None:
            dh_y = torch.zeros_like(c_y)
        dgates, dc_x = gate_ops.lstm_gates_bwd(dh_y, dc_y, act, c_x, c_y)
        return dgates, dgates if ctx.two_products else None, dc_x


class _GruGates(Function):
    """GRU gate arithmetic of one step as one kernel per pass."""

    # pylint: disable=abstract-method, arguments-differ

    @staticmethod
    def forward(ctx, igates: Tensor, hgates: Tensor, h_x: Tensor):
        needs = any(ctx.needs_input_grad)
        hgates, h_x = gate_ops.dense(hgates), gate_ops.dense(h_x)  # the backward pass reads them again
        h_y, act = gate_ops.gru_gates_fwd(igates, hgates, h_x, needs)
        if needs:
            ctx.save_for_backward(act, hgates, h_x)
        return h_y

    @staticmethod
    def backward(ctx, dh_y: Tensor):
        act, hgates, h_x = ctx.saved_tensors
        return gate_ops.gru_gates_bwd(dh_y, act, hgates, h_x)


def lstm_pointwise(igates: Tensor, hgates: Optional[Tensor], c_x: Tensor) -> Tuple[Tensor, Tensor]:
    """``(h_y, c_y)`` from the pre-activations ``[B, 4H]`` of the input product and (if there are
    two products) the hidden product, gate blocks in the order input, forget, cell, output
    (reference cells.py:176-186). One fused kernel where the operands allow it."""
    if gate_ops.gates_supported(igates, hgates, c_x, 4):
        return _LstmGates.apply(igates, hgates, c_x)
    gates = igates if hgates is None else igates + hgates
    in_gate, forget_gate, cell_gate, out_gate = gates.chunk(4, 1)
    c_y = torch.sigmoid(forget_gate) * c_x + torch.sigmoid(in_gate) * torch.tanh(cell_gate)
    return torch.sigmoid(out_gate) * torch.tanh(c_y), c_y


def gru_pointwise(igates: Tensor, hgates: Tensor, h_x: Tensor) -> Tensor:
    """New hidden state from the pre-activations ``[B, 3H]`` of the two products, gate blocks in
    the order reset, update, new; the reset gate scales the hidden part of the candidate after
    the product (reference cells.py:321-343). One fused kernel where the operands allow it."""
    if gate_ops.gates_supported(igates, hgates, h_x, 3):
        return _GruGates.apply(igates, hgates, h_x)
    i_r, i_z, i_n = igates.chunk(3, 1)
    h_r, h_z, h_n = hgates.chunk(3, 1)
    reset = torch.sigmoid(i_r + h_r)
    update = torch.sigmoid(i_z + h_z)
    cand = torch.tanh(i_n + reset * h_n)
    return cand + update * (h_x - cand)


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
        h_y, c_y = lstm_pointwise(igates, self.weight_hh(h_x), c_x)
        return h_y, (h_y, c_y)


class AnalogGRUCell(_AnalogCell):
    """GRU cell, gates stacked as reset, update, new; the reset gate scales the hidden part of
    the candidate after the product, as in ``torch.nn.GRU`` (reference cells.py:270-343)."""

    gate_count = 3

    def recur(self, igates, state):
        h_x, _ = state
        h_y = gru_pointwise(igates, self.weight_hh(h_x), h_x)
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
        h_y, c_y = lstm_pointwise(self.weight(torch.cat((input_, h_x), 1)), None, c_x)
        return h_y, (h_y, c_y)

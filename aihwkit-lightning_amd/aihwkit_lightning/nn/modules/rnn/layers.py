"""One recurrent layer: a cell stepped over the leading (time) dimension, forwards, backwards or
both (reference ``nn/modules/rnn/layers.py:28-183``).

In evaluation mode nothing in an analog product depends on which other rows share the call (the
input range is fixed or per row, no noise is drawn, no statistics are updated), so the input
projection of all time steps is computed as one product over ``steps * batch`` rows, which fills
the GPU where ``batch`` rows per step do not. The result is the same, row for row, as stepping.
In training mode every step calls the cell as the reference does, so that noise draws and
input-range updates happen once per step.
"""
from contextlib import ExitStack
from typing import Any, List, Tuple, Type

import torch
from torch import Tensor
from torch.nn import Module, ModuleList

from ..tiled import TiledAnalogLayer


class AnalogRNNLayer(Module):
    """``cell(*cell_args)`` applied to ``input_[0], input_[1], ...``; the outputs are stacked."""

    time_reversed = False

    def __init__(self, cell: Type, *cell_args: Any):
        super().__init__()
        self.cell = cell(*cell_args)

    def get_zero_state(self, batch_size: int):
        """All-zero state of the cell."""
        return self.cell.get_zero_state(batch_size)

    def _project_ahead(self) -> bool:
        return not self.training and getattr(self.cell, "input_projection_is_separate", False)

    def forward(self, input_: Tensor, state) -> Tuple[Tensor, Any]:
        """``input_ [steps, batch, features]`` -> ``(outputs [steps, batch, hidden], last state)``.
        A reversed layer walks the steps from last to first and returns the outputs in the order
        of the input."""
        steps = input_.size(0)
        order = range(steps - 1, -1, -1) if self.time_reversed else range(steps)
        outputs: List[Tensor] = [None] * steps  # type: ignore[list-item]
        with ExitStack() as stack:
            # the weights do not change between the steps of one sequence
            for module in self.cell.modules():
                if isinstance(module, TiledAnalogLayer):
                    stack.enter_context(module.frozen_weights())
            if self._project_ahead() and steps > 0:
                igates = self.cell.project_input(input_.reshape(steps * input_.size(1), -1))
                igates = igates.view(steps, input_.size(1), -1)
                for t in order:
                    outputs[t], state = self.cell.recur(igates[t], state)
            else:
                for t in order:
                    outputs[t], state = self.cell(input_[t], state)
        return torch.stack(outputs), state


class AnalogReverseRNNLayer(AnalogRNNLayer):
    """The layer of the backward direction."""

    time_reversed = True


class AnalogBidirRNNLayer(Module):
    """A forward and a reversed layer over the same input; outputs concatenated on the feature
    dimension, states returned as a list of two."""

    def __init__(self, cell: Type, *cell_args: Any):
        super().__init__()
        self.directions = ModuleList(
            [AnalogRNNLayer(cell, *cell_args), AnalogReverseRNNLayer(cell, *cell_args)]
        )

    def get_zero_state(self, batch_size: int):
        """Pair of all-zero states."""
        return tuple(d.get_zero_state(batch_size) for d in self.directions)

    def forward(self, input_: Tensor, states) -> Tuple[Tensor, List]:
        """Both directions on ``input_``."""
        results = [d(input_, s) for d, s in zip(self.directions, states)]
        return torch.cat([out for out, _ in results], -1), [s for _, s in results]

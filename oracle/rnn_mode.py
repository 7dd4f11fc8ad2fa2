"""CPU oracle for the recurrent layers -- TEST INFRASTRUCTURE, NOT PRODUCT CODE.

Restates what the reference's ``AnalogRNN`` computes in torch-mode (paths relative to the
reference's ``src/aihwkit_lightning/``): every cell (``nn/modules/rnn/cells.py:45-343``) sends its
input and its hidden state through the AnalogLinear computation and combines the results with
element-wise gate formulas; a layer (``nn/modules/rnn/layers.py:28-183``) steps a cell over the
time dimension forwards, backwards or both; the network (``nn/modules/rnn/rnn.py:41-138``) stacks
layers. Only ``tests/`` may import this module, and only as a checker.

The analog products are the oracle's ``linear_forward`` with its explicit ``linear_backward``,
tied into autograd so that the recurrence is differentiated by torch as in the reference. The
gate formulas are written out here from the textbook definitions; ``tests/test_oracle_rnn.py``
pins them against ``torch.nn.RNN`` / ``LSTM`` / ``GRU`` (independent library routines) with the
non-idealities off, and the whole composition against vectors written by the real reference
(``tests/golden/make_golden_rnn.py``).
"""
from typing import Dict, List, Optional, Sequence, Tuple

import torch
from torch import Tensor

from .torch_mode import OracleCfg, linear_backward, linear_forward


class _AnalogProduct(torch.autograd.Function):
    """``linear_forward`` / ``linear_backward`` as one autograd node."""

    @staticmethod
    def forward(ctx, x, weight, bias, input_range, cfg, training):  # pylint: disable=arguments-differ
        out, saved = linear_forward(x.detach(), weight.detach(),
                                    None if bias is None else bias.detach(), cfg,
                                    None if input_range is None else input_range.detach(), training)
        ctx.saved = saved
        ctx.has = (bias is not None, input_range is not None)
        return out

    @staticmethod
    def backward(ctx, grad_out):  # pylint: disable=arguments-differ
        dx, dw, db, dir_ = linear_backward(grad_out.contiguous(), ctx.saved)
        return dx, dw, db if ctx.has[0] else None, dir_ if ctx.has[1] else None, None, None


class Projection:
    """Parameters of one analog projection: weight ``[N, K]``, bias ``[N]`` or None, input range
    ``[T]`` or None (leaf tensors; gradients accumulate in ``.grad``)."""

    def __init__(self, weight: Tensor, bias: Optional[Tensor], input_range: Optional[Tensor]):
        self.weight = weight.clone().requires_grad_(True)
        self.bias = None if bias is None else bias.clone().requires_grad_(True)
        self.input_range = None if input_range is None else input_range.clone().requires_grad_(True)

    def __call__(self, x: Tensor, cfg: OracleCfg, training: bool) -> Tensor:
        return _AnalogProduct.apply(x, self.weight, self.bias, self.input_range, cfg, training)


def _sigmoid(v: Tensor) -> Tensor:
    return torch.sigmoid(v)


def cell_step(kind: str, proj: Dict[str, Projection], x: Tensor, h: Tensor, c: Optional[Tensor],
              cfg: OracleCfg, training: bool) -> Tuple[Tensor, Optional[Tensor]]:
    """One step of a cell: the new hidden state (= the output) and cell state (LSTM only).

    rnn  (cells.py:96-113):   h' = tanh(Wi x + Wh h)
    lstm (cells.py:168-191):  i, f, g, o = split(Wi x + Wh h); c' = s(f) c + s(i) tanh(g);
                              h' = s(o) tanh(c')
    lstm_combined (cells.py:244-267): the same with one product W [x, h]
    gru  (cells.py:321-343):  r = s(Wi_r x + Wh_r h); z = s(Wi_z x + Wh_z h);
                              n = tanh(Wi_n x + r (Wh_n h)); h' = n + z (h - n)
    """
    if kind == "rnn":
        h_new = torch.tanh(proj["weight_ih"](x, cfg, training) + proj["weight_hh"](h, cfg, training))
        return h_new, None
    if kind in ("lstm", "lstm_combined"):
        if kind == "lstm":
            gates = proj["weight_ih"](x, cfg, training) + proj["weight_hh"](h, cfg, training)
        else:
            gates = proj["weight"](torch.cat((x, h), 1), cfg, training)
        hid = h.size(1)
        i, f = gates[:, :hid], gates[:, hid:2 * hid]
        g, o = gates[:, 2 * hid:3 * hid], gates[:, 3 * hid:]
        c_new = _sigmoid(f) * c + _sigmoid(i) * torch.tanh(g)
        return _sigmoid(o) * torch.tanh(c_new), c_new
    if kind == "gru":
        gi = proj["weight_ih"](x, cfg, training)
        gh = proj["weight_hh"](h, cfg, training)
        hid = h.size(1)
        r = _sigmoid(gi[:, :hid] + gh[:, :hid])
        z = _sigmoid(gi[:, hid:2 * hid] + gh[:, hid:2 * hid])
        n = torch.tanh(gi[:, 2 * hid:] + r * gh[:, 2 * hid:])
        return n + z * (h - n), None
    raise ValueError(kind)


def rnn_forward(kind: str, x: Tensor, cells: Sequence[Dict[str, Projection]], cfg: OracleCfg,
                training: bool, layers: int, bidir: bool,
                states: Optional[Sequence[Tuple[Tensor, Optional[Tensor]]]] = None,
                ) -> Tuple[Tensor, List[Tuple[Tensor, Optional[Tensor]]]]:
    """``x [steps, batch, features]`` through ``layers`` layers (``cells`` in module order: layer
    major, forward direction before the reversed one). Returns the outputs of the last layer
    ``[steps, batch, hidden * directions]`` and the last state of every cell in module order.
    No dropout (the cases use none)."""
    steps, batch = x.shape[:2]
    n_dir = 2 if bidir else 1
    assert len(cells) == layers * n_dir
    last_states = []
    for layer in range(layers):
        per_dir = []
        for d in range(n_dir):
            slot = layer * n_dir + d
            proj = cells[slot]
            hidden = next(iter(proj.values())).weight.size(0) // \
                {"rnn": 1, "lstm": 4, "lstm_combined": 4, "gru": 3}[kind]
            if states is None:
                h = x.new_zeros(batch, hidden)
                c = x.new_zeros(batch, hidden) if kind.startswith("lstm") else None
            else:
                h, c = states[slot]
            outs = [None] * steps
            for t in (range(steps - 1, -1, -1) if d == 1 else range(steps)):
                h, c = cell_step(kind, proj, x[t], h, c, cfg, training)
                outs[t] = h
            per_dir.append(torch.stack(outs))
            last_states.append((h, c))
        x = torch.cat(per_dir, -1)
    return x, last_states
